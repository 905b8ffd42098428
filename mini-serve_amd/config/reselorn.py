"""Typed configuration of the Reselorn decoder, read from its own ``config.json`` keys. The reference has no such
architecture.

``config.json``: ``architecture`` (the name), ``vocab``, ``width``, ``norm.eps`` and ``layers``, a list in which every
entry names its mixer (``type``), the mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``, or null for
none). Layer ``i``'s tensors start with ``l<i>.``.

A layer is ``x += ls1 * N1(mixer(x))``, then ``x += ls2 * N2(ff(x))``: the sublayers read the stream itself, their
output is RMS-normed with a plain weight (``norm1``, ``norm2``) and then scaled per channel (``ls1``, ``ls2``). The mixer:

* ``attention`` (``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, optional ``rot``, ``mask``, ``v_mix``; tensors
  ``mix.q k v o sink vmix``): grouped-query attention. ``rot`` (``base``, ``dims``, optional ``scaling`` with ``factor``,
  ``original``, ``fast``, ``slow``) turns the first ``dims`` elements of each query and key head, halves paired, by
  ``position * base ** (-2i / dims)``; with ``scaling`` the frequencies between the indices at which a wave makes ``fast``
  and ``slow`` turns within ``original`` positions are blended towards ``f / factor`` and cosines and sines are multiplied
  by ``0.1 ln(factor) + 1``. After the rotation every query and key head is divided by its root mean square. A query sees
  the last ``mask.size`` tokens, itself included (no ``mask``: every earlier token); ``exp(sink_h)`` joins head ``h``'s
  softmax denominator. In the layers with ``v_mix`` but the first of them, the values become
  ``(1 - vmix) v + vmix v_first``, ``v_first`` being that first layer's values of the same token; the blend is what
  the cache keeps.

Feed-forwards: ``kind: dense`` (``ff``; tensors ``mlp.gate up down``), ``down(silu(gate x) * up x)``; ``kind: moe``
(``router.experts``, ``router.top``, ``expert.ff``, optional ``shared.ff``; tensors ``mlp.router``, ``mlp.router.b``,
``mlp.e<j>.gate up down``, ``mlp.shared.gate up down``): every token runs the ``top`` experts with the largest router logits
``router x + b``, weighs them by the softmax over those logits alone, and adds the shared expert. The final norm is
``final.norm``; the head is the embedding table ``embed``.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass

from .registry import register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, RunEntry

MIXER_TYPES = ("attention",)
MLP_KINDS = ("dense", "moe")


def _need(d, keys, where: str) -> None:
    if not isinstance(d, dict):
        raise ValueError(f"{where} must be an object, got {d!r}")
    missing = [k for k in keys if k not in d]
    if missing:
        raise KeyError(f"config.json lacks {missing} in {where}")


def _positive_int(d: dict, key: str, where: str) -> int:
    v = d[key]
    if not isinstance(v, int) or isinstance(v, bool) or v < 1:
        raise ValueError(f"{where}.{key} must be a positive integer, got {v!r}")
    return v


@register_architecture("Reselorn")
@dataclass(frozen=True)
class ReselornConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple  # of dicts as in config.json: {"type", "mixer", "mlp"}

    @classmethod
    def from_dict(cls, cfg: dict) -> "ReselornConfig":
        _need(cfg, ("vocab", "width", "norm", "layers"), "config.json")
        _need(cfg["norm"], ("eps",), "norm")
        if not isinstance(cfg["layers"], (list, tuple)) or not cfg["layers"]:
            raise ValueError("layers must be a non-empty list")
        out = cls(
            vocab=_positive_int(cfg, "vocab", "config.json"),
            width=_positive_int(cfg, "width", "config.json"),
            eps=float(cfg["norm"]["eps"]),
            layers=tuple(copy.deepcopy(layer) for layer in cfg["layers"]),
        )
        out.validate()
        return out

    def validate(self) -> None:
        if not self.eps >= 0:
            raise ValueError(f"norm.eps must not be negative, got {self.eps}")
        mixed = None  # (kv_heads, vdim) of the first layer that blends values
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            _need(layer, ("type", "mixer"), where)
            kind, m = layer["type"], layer["mixer"]
            if kind not in MIXER_TYPES:
                raise NotImplementedError(f"{where}.type {kind!r} is not supported, expected one of {MIXER_TYPES}")
            mw = f"{where}.mixer"
            _need(m, ("heads", "kv_heads", "dim", "vdim", "scale"), mw)
            for k in ("heads", "kv_heads", "dim", "vdim"):
                _positive_int(m, k, mw)
            if m["heads"] % m["kv_heads"]:
                raise ValueError(f"{mw}: {m['heads']} heads are no multiple of {m['kv_heads']} kv_heads")
            if not float(m["scale"]) > 0:
                raise ValueError(f"{mw}.scale must be positive")
            rot = m.get("rot")
            if rot:
                _need(rot, ("base", "dims"), f"{mw}.rot")
                dims = rot["dims"]
                if not isinstance(dims, int) or isinstance(dims, bool) or dims % 2 or not 2 <= dims <= m["dim"]:
                    raise ValueError(f"{mw}.rot.dims must be even and at most dim, got {dims!r}")
                if not float(rot["base"]) > 1:
                    raise ValueError(f"{mw}.rot.base must be larger than one")
                sc = rot.get("scaling")
                if sc:
                    _need(sc, ("factor", "original", "fast", "slow"), f"{mw}.rot.scaling")
                    if not (float(sc["factor"]) > 0 and float(sc["original"]) > 0 and float(sc["fast"]) > 0 and float(sc["slow"]) > 0):
                        raise ValueError(f"{mw}.rot.scaling: factor, original, fast and slow must be positive")
            if m.get("mask"):
                _need(m["mask"], ("size",), f"{mw}.mask")
                _positive_int(m["mask"], "size", f"{mw}.mask")
            if m.get("v_mix"):
                shape = (m["kv_heads"], m["vdim"])
                if mixed is None:
                    mixed = shape
                elif shape != mixed:
                    raise ValueError(f"{mw}: values of {shape} (kv_heads, vdim) cannot be blended with the first blending "
                                     f"layer's {mixed}")
            mlp = layer.get("mlp")
            if mlp:
                fw = f"{where}.mlp"
                _need(mlp, ("kind",), fw)
                if mlp["kind"] not in MLP_KINDS:
                    raise NotImplementedError(f"{fw}.kind {mlp['kind']!r} is not supported, expected one of {MLP_KINDS}")
                if mlp["kind"] == "dense":
                    _need(mlp, ("ff",), fw)
                    _positive_int(mlp, "ff", fw)
                else:
                    _need(mlp, ("router", "expert"), fw)
                    _need(mlp["router"], ("experts", "top"), f"{fw}.router")
                    _need(mlp["expert"], ("ff",), f"{fw}.expert")
                    n = _positive_int(mlp["router"], "experts", f"{fw}.router")
                    top = _positive_int(mlp["router"], "top", f"{fw}.router")
                    if top > n:
                        raise ValueError(f"{fw}.router: top {top} of {n} experts")
                    _positive_int(mlp["expert"], "ff", f"{fw}.expert")
                    if mlp.get("shared"):
                        _need(mlp["shared"], ("ff",), f"{fw}.shared")
                        _positive_int(mlp["shared"], "ff", f"{fw}.shared")

    def to_dict(self) -> dict:
        """The ``config.json`` that reads back as this configuration."""
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "layers": [copy.deepcopy(layer) for layer in self.layers]}

    # ------------------------------------------------------------------ lowering

    def _norm(self, tensor: str) -> PartSpec:
        return PartSpec("rmsnorm", {"width": self.width, "eps": self.eps, "tensor": tensor})

    def _mixer(self, m: dict, blend: str | None) -> PartSpec:
        rot, mask = m.get("rot"), m.get("mask")
        position = None
        if rot:
            sc = rot.get("scaling")
            scaling = None if not sc else {"kind": "turn_ramp", "factor": float(sc["factor"]), "original": float(sc["original"]),
                                           "fast": float(sc["fast"]), "slow": float(sc["slow"])}
            position = PartSpec("rotary", {"dim": int(rot["dims"]), "theta": float(rot["base"]), "pairing": "halves",
                                           "scaling": scaling})
        return PartSpec("gqa_attention", {
            "prefix": "mix.", "hidden_size": self.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"],
            "head_dim": m["dim"], "value_dim": m["vdim"], "scale": float(m["scale"]),
            "window": int(mask["size"]) if mask else 0, "qk_norm": "head_rotated", "qk_norm_eps": self.eps,
            "qk_norm_weights": False, "sinks": True, "value_blend": blend, "position": position,
            "names": {"q": "q", "k": "k", "v": "v", "o": "o", "sink": "sink", "blend": "vmix"}})

    def _gated(self, prefix: str, ff: int) -> PartSpec:
        return PartSpec("gated_mlp", {"prefix": prefix, "hidden_size": self.width, "intermediate_size": int(ff),
                                      "activation": "silu", "names": {"gate": "gate", "up": "up", "down": "down"}})

    def _feed_forward(self, mlp: dict | None) -> PartSpec:
        if not mlp:
            return PartSpec("none")
        if mlp["kind"] == "dense":
            return self._gated("mlp.", mlp["ff"])
        shared = mlp.get("shared")
        return PartSpec("moe_mlp", {
            "prefix": "mlp.", "hidden_size": self.width, "intermediate_size": int(mlp["expert"]["ff"]),
            "num_experts": int(mlp["router"]["experts"]), "top": int(mlp["router"]["top"]), "activation": "silu",
            "router_bias": True, "shared": self._gated("mlp.shared.", shared["ff"]) if shared else None,
            "names": {"router": "router", "router_bias": "router.b", "expert": "e{}.", "gate": "gate", "up": "up", "down": "down"}})

    def to_spec(self) -> ModelSpec:
        w = self.width
        layers, order = [], []
        blending = False
        for i, layer in enumerate(self.layers):
            mlp = layer.get("mlp")
            m = layer["mixer"]
            blend = None
            if m.get("v_mix"):
                blend = "blend" if blending else "first"
                blending = True
            block = PartSpec("outnorm", {"mixer_norm": self._norm("norm1"), "ffn_norm": self._norm("norm2") if mlp else None,
                                         "mixer_scale": "ls1", "ffn_scale": "ls2" if mlp else None,
                                         "spare": None if mlp else {"norm2": w, "ls2": w}})
            layers.append(LayerSpec(f"l{i}.", block, self._mixer(m, blend), self._feed_forward(mlp)))
            order.append(RunEntry(i, i))
        return ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab,
            hidden_size=w,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab, "width": w, "tensor": "embed"}),
            layers=tuple(layers),
            run_order=tuple(order),
            final_norm=self._norm("final.norm"),
            head=PartSpec("linear_head", {"vocab_size": self.vocab, "width": w, "tensor": "head", "tied_to": "embed"}),
            max_position=None,
        )
