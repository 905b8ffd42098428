"""Grouped-query softmax attention over the paged cache.

Per layer, in the reference's order (miniserve/model/qwen3.py:110-126): q/k/v projections without
bias, per-head RMSNorm of q and k (one ``[head_dim]`` weight each, shared by all heads), rotation
of q and k, store of k and v into the cache, causal attention in which query head ``h`` reads KV
head ``h // (heads / kv_heads)`` with ``scale`` on the scores, output projection. Here the three
projections are one matrix product over row-concatenated weights (as the reference's fused path
does, miniserve/model/fused.py:204-206); norm, rotation and cache store are one kernel (in a step of
single tokens they are part of the attention kernel); the output
projection adds into the residual stream in its epilogue, or (few rows) leaves partial sums pending
for the next norm to add.

``window > 0`` restricts a query at position p to keys p-window+1 .. p (no counterpart in the
reference). ``qk_norm_eps=None`` switches the per-head norms off; ``position`` may be ``none``.

Further parameters, none of which the reference has (defaults give the layer above):
``keep_first`` (with a window: the sequence's first ``keep_first`` keys stay visible at their true
positions; the cache keeps their pages); ``value_dim`` (size of a value head, default ``head_dim``);
``qk_norm="projection"`` (the RMS norm runs over a token's whole query projection and over its whole key
projection, before they are split into heads, with weights of those sizes; default ``"head"``);
``exact_weights`` (the softmax weights meet the values in float32: no rounding of them to bfloat16 for the
matrix cores); ``names`` (the tensors' names behind the prefix, by ``q k v o q_norm k_norm sink blend q_bias k_bias
v_bias gate``); ``bias`` (the projections have biases, added before anything else); ``values_are_keys`` (there is no
value projection: a token's values are its keys as projected, bias included, before norm and rotation);
``head_gate`` (a tensor ``[heads, hidden]``: head ``h``'s output is multiplied by ``sigmoid(gate x)_h`` before the output
projection). The last three run the path with one norm over the projection.

And four more, which run the path whose every step between projection and attention is a parameter of one kernel
(``ops.head_prepare_store``): ``qk_norm="head_rotated"`` (the norm per head sits behind the rotation instead of before
it: with cosines and sines that carry a magnitude the two differ); ``qk_norm_weights=False`` (the norms have no weights:
a bare division by the root mean square); ``sinks`` (a learned number per query head, tensor ``[heads]``, whose exponential
joins the head's softmax denominator with neither key nor value); ``value_blend`` (``"first"``: the layer's values, as
projected, are kept for the step's later layers; ``"blend"``: its values become ``(1 - a) v + a v_first`` with the one
learned number ``a`` (tensor ``[]``) and ``v_first`` the values of the same token that the ``"first"`` layer of the same
``blend_group`` kept; the blend is what is cached and attended over. The two layers' value shapes must agree).
"""

from __future__ import annotations

import warnings

import torch

from ..config.spec import PartSpec
from .base import KVNeed, Mixer, TensorSpec
from .registry import part_class, register


def _names(spec: PartSpec) -> dict[str, str]:
    p = spec.get("prefix", "")
    given = spec.get("names") or {}
    default = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
               "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", "sink": "sinks", "blend": "value_blend",
               "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "gate": "gate.weight"}
    return {k: p + given.get(k, d) for k, d in default.items()}


@register("mixer", "gqa_attention")
class GQAttention(Mixer):
    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.prefix = spec.get("prefix", "")
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.kv_heads = int(spec["num_kv_heads"])
        self.head_dim = int(spec["head_dim"])
        self.scale = float(spec["scale"])
        self.qk_norm_eps = spec.get("qk_norm_eps")
        self.window = int(spec.get("window") or 0)
        self.keep_first = int(spec.get("keep_first") or 0) if self.window else 0
        self.value_dim = int(spec.get("value_dim") or self.head_dim)
        self.qk_norm = spec.get("qk_norm", "head")
        self.exact_weights = bool(spec.get("exact_weights", False))
        self.names = _names(spec)
        self.qk_norm_weights = bool(spec.get("qk_norm_weights", True))
        self.sinks = bool(spec.get("sinks", False))
        self.value_blend = spec.get("value_blend")
        self.blend_key = ("value_blend", spec.get("blend_group", "values"))
        self.bias = bool(spec.get("bias", False))
        self.values_are_keys = bool(spec.get("values_are_keys", False))
        self.head_gate = bool(spec.get("head_gate", False))
        if self.values_are_keys and self.value_dim != self.head_dim:
            raise ValueError(f"values that are the keys have the keys' size {self.head_dim}, not {self.value_dim}")
        if self.qk_norm not in ("head", "projection", "head_rotated"):
            raise ValueError(f"qk_norm {self.qk_norm!r}: 'head', 'projection' or 'head_rotated'")
        if self.value_blend not in (None, "first", "blend"):
            raise ValueError(f"value_blend {self.value_blend!r}: None, 'first' or 'blend'")
        # The path on which rotation, norm, blend and store are one kernel with every option a parameter.
        self.prepared = (self.qk_norm == "head_rotated" or self.sinks or self.value_blend is not None
                         or (self.qk_norm_eps is not None and not self.qk_norm_weights))
        if self.prepared and (self.qk_norm == "projection" or self.keep_first):
            raise NotImplementedError("sinks, blended values and a norm behind the rotation go with a norm per head and no kept first keys")
        extras = self.bias or self.values_are_keys or self.head_gate
        if extras and (self.prepared or (self.qk_norm == "head" and self.qk_norm_eps is not None)):
            raise NotImplementedError("biases, values that are the keys and a gate per head go with one norm over the projection or none")
        if self.keep_first < 0 or self.window < 0:
            raise ValueError("window and keep_first must not be negative")
        # The path with one norm over the projection, values of their own size, kept first keys or unrounded weights.
        self.wide = not self.prepared and ((self.qk_norm == "projection" and self.qk_norm_eps is not None)
                                           or self.value_dim != self.head_dim or extras)
        if self.wide and self.qk_norm == "head" and self.qk_norm_eps is not None:
            raise NotImplementedError("a norm per head together with values of another size than the keys is not supported")
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} query heads are no multiple of {self.kv_heads} KV heads")
        # What the attention kernels refuse is refused here, when the model is built, not in its first step.
        limit = 1024 if self.sinks else 256  # what the kernels that know sinks take
        if not (1 <= self.head_dim <= limit and 1 <= self.value_dim <= limit):
            raise ValueError(f"head sizes {self.head_dim} / {self.value_dim} are not supported: the attention kernels take sizes up to {limit}")
        if not self.scale > 0:
            raise ValueError(f"the attention scale must be positive, not {self.scale}")
        generic = self.wide or self.exact_weights or self.keep_first or self.prepared
        if rt is not None and rt.dtype == torch.bfloat16 and not generic and not (
                self.head_dim in (64, 128) and self.heads // self.kv_heads <= 16):
            warnings.warn(
                f"attention with head_dim {self.head_dim} and {self.heads // self.kv_heads} query heads per KV head runs the "
                "generic kernel in bfloat16 (one wave per token and head): the matrix-core kernels take head sizes 64 and 128 "
                "with up to 16 query heads per KV head", stacklevel=2)
        pos = spec.get("position") or PartSpec("none")
        self.position = part_class("position", pos)(pos, rt)
        self.qkv = self.o = self.q_norm = self.k_norm = self.sink = self.qkv_bias = None
        self.blend = 0.0
        self.gate_col = 0

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        n = _names(spec)
        h, d = int(spec["hidden_size"]), int(spec["head_dim"])
        dv = int(spec.get("value_dim") or d)
        hq, hkv = int(spec["num_heads"]), int(spec["num_kv_heads"])
        own_values = not spec.get("values_are_keys", False)
        out = {
            n["q"]: TensorSpec((hq * d, h)),
            n["k"]: TensorSpec((hkv * d, h)),
            n["o"]: TensorSpec((h, hq * dv)),
        }
        if own_values:
            out[n["v"]] = TensorSpec((hkv * dv, h))
        if spec.get("bias", False):
            out[n["q_bias"]] = TensorSpec((hq * d,), init="uniform")
            out[n["k_bias"]] = TensorSpec((hkv * d,), init="uniform")
            if own_values:
                out[n["v_bias"]] = TensorSpec((hkv * dv,), init="uniform")
        if spec.get("head_gate", False):
            out[n["gate"]] = TensorSpec((hq, h))
        if spec.get("qk_norm_eps") is not None and spec.get("qk_norm_weights", True):
            whole = spec.get("qk_norm", "head") == "projection"
            out[n["q_norm"]] = TensorSpec((hq * d if whole else d,), init="ones")
            out[n["k_norm"]] = TensorSpec((hkv * d if whole else d,), init="ones")
        if spec.get("sinks", False):
            out[n["sink"]] = TensorSpec((hq,), init="uniform")
        if "blend" in (spec.get("names") or {}) or spec.get("value_blend") == "blend":
            # one number; a layer that does not blend may still carry it, and nothing reads it there
            out[n["blend"]] = TensorSpec((), init="uniform", optional=spec.get("value_blend") != "blend")
        return out

    def bind(self, tensors) -> None:
        p, n = self.prefix, self.names
        kinds = ("q", "k") if self.values_are_keys else ("q", "k", "v")
        parts = [tensors[n[k]] for k in kinds]
        if self.bias:
            biases = [tensors[n[k + "_bias"]] for k in kinds]
            if len({t.dtype for t in biases}) != 1:
                raise ValueError(f"{p}the projections' biases are stored in different dtypes")
            self.qkv_bias = torch.cat(biases, dim=0).contiguous()
        if self.head_gate:
            self.gate_col = sum(t.shape[0] for t in parts)  # the gate's rows lie behind the projections
            parts.append(tensors[n["gate"]])
        if len({t.dtype for t in parts}) != 1:
            raise ValueError(f"{p}q/k/v projections are stored in different dtypes")
        self.qkv = torch.cat(parts, dim=0).contiguous()
        self.o = tensors[n["o"]]
        if self.qk_norm_eps is not None and self.qk_norm_weights:
            self.q_norm = tensors[n["q_norm"]]
            self.k_norm = tensors[n["k_norm"]]
        if self.sinks:
            self.sink = tensors[n["sink"]].to(torch.float32).contiguous()
        if self.value_blend == "blend":
            self.blend = float(tensors[n["blend"]].to(torch.float32).item())  # one number, read once

    def kv_need(self) -> KVNeed:
        return KVNeed.keys_values(self.kv_heads, self.head_dim, self.window, self.value_dim, self.keep_first)

    def forward(self, x, batch, cache, state, residual):
        ops = self.rt.ops
        rot = self.position.rotation(batch)
        table = rot.table if rot is not None else None
        pairing = rot.pairing if rot is not None else "halves"
        eps = 0.0 if self.qk_norm_eps is None else float(self.qk_norm_eps)
        if self.prepared:
            return self._forward_prepared(x, batch, cache, residual, table, pairing, eps)
        if self.wide:
            qkv = ops.linear(x, self.qkv, out_dtype=torch.float32)  # the norms' input is not rounded
            q = ops.qkv_norm_rope_store(qkv, cache.slots if cache.writes else None, self.q_norm, self.k_norm, eps, table,
                                        cache.k, cache.v, self.heads, self.kv_heads, self.head_dim, self.value_dim,
                                        self.rt.dtype, pairing, self.qkv_bias, self.values_are_keys, self.heads if self.head_gate else 0)
            out = ops.paged_attention(q, cache.k, cache.v, cache.block_table, batch, self.heads, self.kv_heads, self.head_dim,
                                      self.scale, self.window, self.value_dim, self.keep_first, self.exact_weights)
            if self.head_gate:
                ops.head_gate_(out, qkv, self.gate_col, self.heads)
            return ops.linear(out, self.o, accumulate_into=residual, defer=True)
        qkv = ops.linear(x, self.qkv, out_dtype=self.rt.dtype, defer=True)
        if not (self.exact_weights or self.keep_first) and ops.decode_attention_fusable(qkv, batch, self.q_norm, self.k_norm, table, cache.k, cache.v,
                                        self.heads, self.kv_heads, self.head_dim, pairing):
            # a step of single tokens: norm, rotation, cache store and attention are one kernel
            # ... and, with few rows, the reduction of the key splits and the output projection another
            out = ops.decode_attention_fused(
                qkv, self.q_norm, self.k_norm, 0.0 if self.qk_norm_eps is None else float(self.qk_norm_eps), table,
                cache.writes, cache.k, cache.v, cache.block_table, batch, self.heads, self.kv_heads, self.head_dim,
                self.scale, self.window, project=self.o if self.o.dtype == torch.bfloat16 else None,
            )
            if isinstance(out, ops.SplitSum):
                return out  # the projection's partial sums: pending, for the next reader of the stream
            return ops.linear(out, self.o, accumulate_into=residual, defer=True)
        q = ops.qk_norm_rope_store(
            qkv, cache.slots if cache.writes else None,
            self.q_norm, self.k_norm, 0.0 if self.qk_norm_eps is None else float(self.qk_norm_eps),
            table,
            cache.k, cache.v, self.heads, self.kv_heads, self.head_dim, out_dtype=self.rt.dtype, pairing=pairing,
        )
        out = ops.paged_attention(
            q, cache.k, cache.v, cache.block_table, batch, self.heads, self.kv_heads, self.head_dim,
            self.scale, self.window, None, self.keep_first, self.exact_weights,
        )
        return ops.linear(out, self.o, accumulate_into=residual, defer=True)

    def _forward_prepared(self, x, batch, cache, residual, table, pairing, eps):
        ops = self.rt.ops
        qkv = ops.linear(x, self.qkv, out_dtype=torch.float32)  # what norms and blends read is not rounded
        v_first = None
        if self.value_blend is not None:
            if not cache.writes:
                raise NotImplementedError("a layer that blends values keeps keys and values of its own")
            if self.value_blend == "first":
                # a view of this step's projection: the values as projected, one row per token
                batch.memo[self.blend_key] = qkv[:, (self.heads + self.kv_heads) * self.head_dim:]
            else:
                v_first = batch.memo.get(self.blend_key)
                if v_first is None:
                    raise ValueError(f"no earlier layer of the step kept values for {self.blend_key[1]!r}")
                if v_first.shape[1] != self.kv_heads * self.value_dim:
                    raise ValueError(f"values of width {self.kv_heads * self.value_dim} cannot be blended with kept values of "
                                     f"width {v_first.shape[1]}")
        norm = None if self.qk_norm_eps is None else ("after" if self.qk_norm == "head_rotated" else "before")
        q = ops.head_prepare_store(qkv, cache.slots if cache.writes else None, norm, self.q_norm, self.k_norm, eps, table, pairing,
                                   cache.k, cache.v, self.heads, self.kv_heads, self.head_dim, self.value_dim, self.rt.dtype,
                                   v_first, self.blend)
        out = ops.paged_attention(q, cache.k, cache.v, cache.block_table, batch, self.heads, self.kv_heads, self.head_dim,
                                  self.scale, self.window, self.value_dim, sinks=self.sink)
        return ops.linear(out, self.o, accumulate_into=residual, defer=True)

    def parameters_bytes(self) -> int:
        ts = [self.qkv, self.o] + ([self.q_norm, self.k_norm] if self.q_norm is not None else []) + [
            t for t in (self.sink, self.qkv_bias) if t is not None]
        return sum(t.numel() * t.element_size() for t in ts)

    def flops(self, rows) -> int:
        """The four projections, and both attention products over every (query, visible key) pair: a query
        at position p sees keys ``max(0, p - window + 1) .. p`` and the kept first keys."""
        tokens = sum(n for n, _ in rows)
        pairs = 0
        for n, cached in rows:
            for p in (range(cached, cached + n) if self.window else ()):
                pairs += min(p + 1, self.window + self.keep_first)
            if not self.window:
                pairs += n * cached + n * (n + 1) // 2
        qk, vo = self.heads * self.head_dim, self.heads * self.value_dim
        projected = qk + self.kv_heads * (self.head_dim + (0 if self.values_are_keys else self.value_dim)) + (self.heads if self.head_gate else 0)
        linear = 2 * tokens * self.hidden * projected + 2 * tokens * vo * self.hidden
        return linear + 2 * pairs * (qk + vo)
