"""RMSNorm: ``y = w * x * rsqrt(mean(x^2) + eps)``, statistics and scaling in float32, plain weight
(not ``1 + w``) as in the reference (miniserve/model/qwen3.py:78-82). The reference rounds to the
model dtype before the weight product; here the whole expression is evaluated in float32 and
rounded once, which is what its fused operators do (miniserve/model/fused.py:188-194).

``offset`` (optional, no counterpart in the reference): the stored weight lies around zero and the norm multiplies by
``offset + w`` (``offset = 1``: the "one plus weight" form). The sum is formed once, in float32, when the weight is bound.
``fold_scale`` lets a block hang a scale per channel behind the norm (a layer scale) at no cost per step."""

from __future__ import annotations

import torch

from ..config.spec import PartSpec
from .base import Norm, TensorSpec
from .registry import register


@register("norm", "rmsnorm")
class RMSNorm(Norm):
    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.width = int(spec["width"])
        self.eps = float(spec["eps"])
        self.offset = float(spec.get("offset") or 0.0)
        self.weight = None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        # a weight stored around zero is drawn around zero
        return {spec["tensor"]: TensorSpec((int(spec["width"]),), init="uniform" if spec.get("offset") else "ones")}

    def bind(self, tensors) -> None:
        self.weight = tensors[self.spec["tensor"]]
        if self.offset:
            self.weight = (self.weight.to(torch.float32) + self.offset).contiguous()

    def fold_scale(self, scale) -> None:
        """Multiply what the norm puts out by ``scale [width]``, element by element: the product with the weight is
        formed once, in float32 (two bfloat16 numbers multiply exactly there), and takes the weight's place."""
        self.weight = (self.weight.to(torch.float32) * scale.to(torch.float32)).contiguous()

    def forward(self, x, rows=None, add=None):
        """``x``: float32 ``[T, width]``; ``rows``: optional int32 row indices to normalise (the
        others are skipped); ``add``: a pending sum added into the normalised rows of ``x`` first.
        Returns the compute dtype, ``[T or len(rows), width]``."""
        return self.rt.ops.rmsnorm(x, self.weight, self.eps, self.rt.dtype, rows, add)

    def add_normed(self, residual, stream, pending=None, next_out=None, clear=False) -> None:
        """``residual += norm(stream + pending)``; ``next_out`` (bfloat16) receives the new residual rounded, and with
        ``clear`` the stream is left zero (both inside the norm's kernel)."""
        self.rt.ops.normed_add(residual, stream, self.weight, self.eps, pending, next_out, clear)

    def parameters_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()


@register("norm", "layernorm")
class LayerNorm(Norm):
    """``y = (x - mean(x)) / sqrt(var(x) + eps) * w + b``, the variance being the mean of the squared
    deviations; statistics and scaling in float32. ``bias_tensor`` names the bias (None: no bias)."""

    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.width = int(spec["width"])
        self.eps = float(spec["eps"])
        self.weight = self.bias = None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        out = {spec["tensor"]: TensorSpec((int(spec["width"]),), init="ones")}
        if spec.get("bias_tensor"):
            out[spec["bias_tensor"]] = TensorSpec((int(spec["width"]),), init="uniform")
        return out

    def bind(self, tensors) -> None:
        self.weight = tensors[self.spec["tensor"]]
        self.bias = tensors[self.spec["bias_tensor"]] if self.spec.get("bias_tensor") else None

    def forward(self, x, rows=None, add=None):
        ops = self.rt.ops
        ops.add_pending(x, add)  # the kernel takes no pending sum along: the stream is brought up to date first
        return ops.layernorm(x, self.weight, self.bias, self.eps, self.rt.dtype, rows)

    def parameters_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.weight, self.bias) if t is not None)
