"""Block arrangements: where the norms and the residual sums sit around a mixer and a
feed-forward. ``prenorm`` is the reference's (miniserve/model/qwen3.py:212-216):
``h += mixer(norm(h)); h += feed_forward(norm(h))``. ``parallel``, ``outnorm`` and ``sandwich`` have no counterpart there."""

from __future__ import annotations

import torch

from ..config.spec import PartSpec
from .base import ROUNDED_RESIDUAL, Block, TensorSpec
from .registry import part_class, register


@register("block", "prenorm")
class PreNormBlock(Block):
    def __init__(self, spec: PartSpec, rt, mixer, feed_forward):
        super().__init__(spec, rt, mixer, feed_forward)
        mn, fn = spec["mixer_norm"], spec["ffn_norm"]
        self.mixer_norm = part_class("norm", mn)(mn, rt)
        self.ffn_norm = part_class("norm", fn)(fn, rt)

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        out = {}
        for key in ("mixer_norm", "ffn_norm"):
            s = spec[key]
            out.update(part_class("norm", s).tensors(s))
        return out

    def bind(self, tensors) -> None:
        self.mixer_norm.bind(tensors)
        self.ffn_norm.bind(tensors)

    def forward(self, residual, batch, cache, state, pending=None):
        x = self.mixer_norm.forward(residual, add=pending)
        pending = self.mixer.forward(x, batch, cache, state, residual)
        y = self.ffn_norm.forward(residual, add=pending)
        return self.feed_forward.forward(y, residual)

    def parameters_bytes(self) -> int:
        return self.mixer_norm.parameters_bytes() + self.ffn_norm.parameters_bytes()


@register("block", "parallel")
class ParallelBlock(Block):
    """``h += mixer(norm(h)) + feed_forward(norm(h))``: one norm, both sublayers read its output."""

    def __init__(self, spec: PartSpec, rt, mixer, feed_forward):
        super().__init__(spec, rt, mixer, feed_forward)
        n = spec["norm"]
        self.norm = part_class("norm", n)(n, rt)

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        return part_class("norm", spec["norm"]).tensors(spec["norm"])

    def bind(self, tensors) -> None:
        self.norm.bind(tensors)

    def forward(self, residual, batch, cache, state, pending=None):
        x = self.norm.forward(residual, add=pending)
        first = self.mixer.forward(x, batch, cache, state, residual)
        second = self.feed_forward.forward(x, residual)
        if first is not None and second is not None:
            self.rt.ops.add_pending(residual, first)
            return second
        return first if first is not None else second

    def parameters_bytes(self) -> int:
        return self.norm.parameters_bytes()


@register("block", "outnorm")
class OutputNormBlock(Block):
    """``h += norm1(mixer(h)); h += norm2(feed_forward(h))``: the sublayers read the stream itself, and what they put
    out is normed before it joins the stream. Each sublayer adds into a stream that starts at zero; the norm's
    ``add_normed`` folds it into the residual stream and leaves it zero for the next sublayer. A layer without a feed-forward has no second norm
    (``ffn_norm`` None); ``spare`` then names norm tensors ``{name: width}`` that a checkpoint may still carry for it.
    ``mixer_scale`` / ``ffn_scale`` (optional) name a tensor ``[width]`` each by which the normed output is multiplied
    element by element before it joins the stream (a layer scale): ``h += scale * norm(sublayer(h))``. It is folded into
    the norm's weight when the tensors are bound."""

    def __init__(self, spec: PartSpec, rt, mixer, feed_forward):
        super().__init__(spec, rt, mixer, feed_forward)
        mn, fn = spec["mixer_norm"], spec.get("ffn_norm")
        self.mixer_norm = part_class("norm", mn)(mn, rt)
        self.ffn_norm = part_class("norm", fn)(fn, rt) if fn is not None else None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        out = {}
        for key in ("mixer_norm", "ffn_norm"):
            s = spec.get(key)
            if s is not None:
                out.update(part_class("norm", s).tensors(s))
        for key, norm in (("mixer_scale", "mixer_norm"), ("ffn_scale", "ffn_norm")):
            if spec.get(key) and spec.get(norm) is not None:
                out[spec[key]] = TensorSpec((int(spec[norm]["width"]),), init="ones")
        for name, width in (spec.get("spare") or {}).items():
            out[name] = TensorSpec((int(width),), optional=True)
        return out

    def bind(self, tensors) -> None:
        self.mixer_norm.bind(tensors)
        if self.spec.get("mixer_scale"):
            self.mixer_norm.fold_scale(tensors[self.spec["mixer_scale"]])
        if self.ffn_norm is not None:
            self.ffn_norm.bind(tensors)
            if self.spec.get("ffn_scale"):
                self.ffn_norm.fold_scale(tensors[self.spec["ffn_scale"]])

    def forward(self, residual, batch, cache, state, pending=None):
        ops, dtype = self.rt.ops, self.rt.dtype
        ops.add_pending(residual, pending)
        # The stream the sublayers add into is zeroed once per pass: the norm's kernel leaves it zero again. The same
        # kernel hands the next reader (the feed-forward, the next block) the new residual in the compute dtype, so that
        # a layer casts the stream only where the block before it left no such copy.
        key = ("outnorm_stream", tuple(residual.shape))
        own = batch.memo.get(key)
        if own is None:
            own = batch.memo[key] = torch.zeros_like(residual)
        rounded = dtype == torch.bfloat16
        x = batch.memo.pop(ROUNDED_RESIDUAL, None)
        if pending is not None or x is None or x.shape != residual.shape or x.dtype != dtype:
            x = ops.cast(residual, dtype)
        first = self.mixer.forward(x, batch, cache, state, own)
        x = torch.empty_like(x) if rounded else residual
        self.mixer_norm.add_normed(residual, own, first, next_out=x if rounded else None, clear=True)
        if self.ffn_norm is not None:
            second = self.feed_forward.forward(x, own)
            x = torch.empty_like(x) if rounded else residual
            self.ffn_norm.add_normed(residual, own, second, next_out=x if rounded else None, clear=True)
        if rounded:
            batch.memo[ROUNDED_RESIDUAL] = x
        return None

    def parameters_bytes(self) -> int:
        return self.mixer_norm.parameters_bytes() + (self.ffn_norm.parameters_bytes() if self.ffn_norm is not None else 0)


@register("block", "sandwich")
class SandwichBlock(Block):
    """``h += out1(mixer(in1(h))); h += out2(feed_forward(in2(h)))``: a norm in front of every sublayer and another
    behind it. The norms in front are the pre-norm block's (``mixer_norm``, ``ffn_norm``), the ones behind the
    output-norm block's (``mixer_out_norm``, ``ffn_out_norm``): each sublayer adds into a stream that starts at zero,
    and the norm behind it folds that stream into the residual stream and leaves it zero again. A layer without a
    feed-forward has neither ``ffn_norm`` nor ``ffn_out_norm`` (None); ``spare`` then names norm tensors
    ``{name: width}`` that a checkpoint may still carry for them."""

    NORMS = ("mixer_norm", "mixer_out_norm", "ffn_norm", "ffn_out_norm")

    def __init__(self, spec: PartSpec, rt, mixer, feed_forward):
        super().__init__(spec, rt, mixer, feed_forward)
        if (spec.get("ffn_norm") is None) != (spec.get("ffn_out_norm") is None):
            raise ValueError("the feed-forward's two norms come together or not at all")
        self.norms = {k: part_class("norm", spec[k])(spec[k], rt) if spec.get(k) is not None else None for k in self.NORMS}

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        out = {}
        for key in cls.NORMS:
            s = spec.get(key)
            if s is not None:
                out.update(part_class("norm", s).tensors(s))
        for name, width in (spec.get("spare") or {}).items():
            out[name] = TensorSpec((int(width),), optional=True)
        return out

    def bind(self, tensors) -> None:
        for n in self.norms.values():
            if n is not None:
                n.bind(tensors)

    def forward(self, residual, batch, cache, state, pending=None):
        n = self.norms
        key = ("outnorm_stream", tuple(residual.shape))  # one zeroed stream per pass, shared with the output-norm blocks
        own = batch.memo.get(key)
        if own is None:
            own = batch.memo[key] = torch.zeros_like(residual)
        batch.memo.pop(ROUNDED_RESIDUAL, None)  # the norm in front reads the stream itself
        x = n["mixer_norm"].forward(residual, add=pending)
        first = self.mixer.forward(x, batch, cache, state, own)
        n["mixer_out_norm"].add_normed(residual, own, first, clear=True)
        if n["ffn_norm"] is not None:
            y = n["ffn_norm"].forward(residual)
            second = self.feed_forward.forward(y, own)
            n["ffn_out_norm"].add_normed(residual, own, second, clear=True)
        return None

    def parameters_bytes(self) -> int:
        return sum(n.parameters_bytes() for n in self.norms.values() if n is not None)
