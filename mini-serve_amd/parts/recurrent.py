"""Mixers that keep a matrix state of fixed size per request and head instead of keys and values per token,
and the mixer that runs two mixers side by side. None has a counterpart in the reference.

Both recurrent mixers are ``S_t = a_t S_(t-1) + b_t k_t v_t^T``, ``o_t = S_t^T q_t`` per head (``S: [dim, value_dim]``),
computed in float32 by one kernel family (``ops.gated_recurrence``) whose state lives in the cache manager's state
slots; they differ in where ``a`` and ``b`` come from and in what happens to ``o``:

* ``decay_linear_attention``: ``q, k, v = silu(W h)``; ``a`` is a constant per head (``decay``), ``b = 1``; the
  concatenated heads are RMS-normed together (weight ``norm``), multiplied by ``sigmoid(W_g h)`` and projected.
  Options, whose defaults give that layer: ``activation`` (``"silu"`` or None: q, k, v as projected), ``position`` (a
  position encoding that turns q and k, in float32, before the recurrence), ``k_scale`` (k is multiplied by it, behind
  the rotation), ``norm_group`` (``"row"``: one norm over the concatenated heads; ``"head"``: one per head),
  ``norm_weight`` (False: a bare division by the root mean square, no ``norm`` tensor), ``gate_activation``
  (``"sigmoid"`` or ``"silu"``).
* ``mlstm``: ``q = W_q h / sqrt(dim)``, ``k``, ``v`` plain; a log input gate and a log forget gate per head, each
  bounded by a soft cap (``cap tanh(z / cap)``, the forget gate then through a log-sigmoid), a running maximum that
  keeps the exponentials in range, and a normaliser vector ``n``; each head's output is divided by its root mean
  square, the heads are concatenated, multiplied by a weight and by ``sigmoid(W_g h)`` and projected.

All projections of a mixer are one matrix product over row-concatenated weights whose float32 result the recurrence
kernel reads in place (activation, scale and gates are applied on the way in).

* ``wkv``: the same state with a decay per key channel and token and a bonus for the current token,
  ``o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t``, then ``S_t = diag(w_t) S_(t-1) + k_t v_t^T``. Each of r, k, v, the gate and
  the decay reads its own blend of the token's input and the previous token's, ``h + (h' - h) mu_s`` (``h' = 0`` for a
  sequence's first token; a request's last input is part of its state); ``w = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0))``;
  each head's output is divided by its root mean square, the heads are concatenated, multiplied by a weight and by
  ``silu(W_g mix_g)`` and projected. Its five products read five different inputs, so they stay five products; they
  write into the columns of one float32 matrix that the kernels behind them read side by side.
"""

from __future__ import annotations

import torch

from ..config.spec import PartSpec
from .base import KVNeed, Mixer, StateNeed, StateTensor, TensorSpec
from .registry import part_class, register


def _named(spec: PartSpec, default: dict) -> dict[str, str]:
    p = spec.get("prefix", "")
    given = spec.get("names") or {}
    return {k: p + given.get(k, d) for k, d in default.items()}


class _RecurrentMixer(Mixer):
    """What the two recurrent mixers share: sizes, the fused projection and the gated output norm."""

    NAMES: dict = {}

    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.dim = int(spec["head_dim"])
        self.value_dim = int(spec.get("value_dim") or self.dim)
        self.eps = float(spec["eps"])
        self.names = _named(spec, self.NAMES)
        if min(self.heads, self.dim, self.value_dim) < 1 or max(self.dim, self.value_dim) > 256:
            raise ValueError(f"{self.heads} heads of sizes {self.dim} / {self.value_dim}: the recurrence kernels take sizes 1..256")
        self.proj = self.o = self.norm = None
        self.columns: dict[str, int] = {}

    def _fuse(self, tensors, order) -> None:
        parts = [tensors[self.names[k]] for k in order]
        if len({t.dtype for t in parts}) != 1:
            raise ValueError(f"{self.names[order[0]]} and its neighbours are stored in different dtypes")
        at = 0
        for k, t in zip(order, parts):
            self.columns[k] = at
            at += t.shape[0]
        self.proj = torch.cat(parts, dim=0).contiguous()
        self.o = tensors[self.names["o"]]
        self.norm = tensors[self.names["norm"]] if self.names["norm"] in tensors else None

    def _finish(self, o, x32, group, residual, gate_activation: str = "sigmoid"):
        ops = self.rt.ops
        n = self.heads * self.value_dim
        gate = x32[:, self.columns["g"] : self.columns["g"] + n]
        y = ops.group_rmsnorm_gate(o, group, self.norm, gate, self.eps, self.rt.dtype, gate_activation)
        return ops.linear(y, self.o, accumulate_into=residual, defer=True)

    def parameters_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.proj, self.o, self.norm) if t is not None)

    def flops(self, rows) -> int:
        tokens = sum(n for n, _ in rows)
        qk, vo = self.heads * self.dim, self.heads * self.value_dim
        linear = 2 * tokens * self.hidden * (self.proj.shape[0] if self.proj is not None else 2 * qk + 2 * vo) + 2 * tokens * vo * self.hidden
        return linear + 4 * tokens * self.heads * self.dim * self.value_dim  # the state's update and its product with q


@register("mixer", "decay_linear_attention")
class DecayLinearAttention(_RecurrentMixer):
    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm"}

    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        decay = [float(d) for d in spec["decay"]]
        if len(decay) != self.heads:
            raise ValueError(f"{len(decay)} decays for {self.heads} heads")
        if not all(0.0 <= d <= 1.0 for d in decay):
            raise ValueError(f"decays must lie in [0, 1], got {decay}")
        self.decay = torch.tensor(decay, dtype=torch.float32, device=rt.device) if rt is not None else None
        self.chunks = min(decay) > 1e-30  # the chunked kernels work with the decays' logarithms
        self.activation = spec.get("activation", "silu")
        self.k_scale = float(spec.get("k_scale", 1.0))
        self.norm_group = spec.get("norm_group", "row")
        self.gate_activation = spec.get("gate_activation", "sigmoid")
        if self.activation not in (None, "silu"):
            raise NotImplementedError(f"activation {self.activation!r} of q, k and v: None or 'silu'")
        if self.norm_group not in ("row", "head"):
            raise ValueError(f"norm_group {self.norm_group!r}: 'row' or 'head'")
        if rt is not None and self.gate_activation not in rt.ops.GATE_ACTIVATIONS:
            raise NotImplementedError(f"gate activation {self.gate_activation!r}: one of {sorted(rt.ops.GATE_ACTIVATIONS)}")
        pos = spec.get("position") or PartSpec("none")
        self.position = part_class("position", pos)(pos, rt)

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        n = _named(spec, cls.NAMES)
        w, h, d = int(spec["hidden_size"]), int(spec["num_heads"]), int(spec["head_dim"])
        e = int(spec.get("value_dim") or d)
        out = {n["q"]: TensorSpec((h * d, w)), n["k"]: TensorSpec((h * d, w)), n["v"]: TensorSpec((h * e, w)),
               n["g"]: TensorSpec((h * e, w)), n["o"]: TensorSpec((w, h * e))}
        if spec.get("norm_weight", True):
            out[n["norm"]] = TensorSpec((h * e,), init="ones")
        return out

    def bind(self, tensors) -> None:
        self._fuse(tensors, ("q", "k", "v", "g"))

    def state_need(self) -> StateNeed:
        return StateNeed((StateTensor("S", (self.heads, self.dim, self.value_dim), "float32"),))

    def forward(self, x, batch, cache, state, residual):
        ops = self.rt.ops
        x32 = ops.linear(x, self.proj, out_dtype=torch.float32)
        rot = self.position.rotation(batch)
        if rot is not None or self.k_scale != 1.0:
            if rot is not None and self.activation is not None:
                raise NotImplementedError("a rotation of q and k goes with q and k as projected (activation None)")
            table, pairing = (rot.table, rot.pairing) if rot is not None else (None, "halves")
            ops.rotate_columns_(x32, self.columns["q"], self.heads, self.dim, table, pairing, 1.0)
            ops.rotate_columns_(x32, self.columns["k"], self.heads, self.dim, table, pairing, self.k_scale)
        o = ops.gated_recurrence(x32, self.columns, self.heads, self.dim, self.value_dim, batch, state, mode="decay",
                                 activation=self.activation, decay=self.decay, chunks=self.chunks)
        group = self.value_dim if self.norm_group == "head" else self.heads * self.value_dim
        return self._finish(o, x32, group, residual, self.gate_activation)


@register("mixer", "mlstm")
class MLSTM(_RecurrentMixer):
    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "i": "i", "f": "f", "i_bias": "i.b", "f_bias": "f.b", "o": "o",
             "norm": "norm"}

    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.cap = float(spec["gate_cap"])
        if not self.cap > 0:
            raise ValueError(f"gate_cap must be positive, not {self.cap}")
        self.i_bias = self.f_bias = None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        n = _named(spec, cls.NAMES)
        w, h, d = int(spec["hidden_size"]), int(spec["num_heads"]), int(spec["head_dim"])
        e = int(spec.get("value_dim") or d)
        return {n["q"]: TensorSpec((h * d, w)), n["k"]: TensorSpec((h * d, w)), n["v"]: TensorSpec((h * e, w)),
                n["g"]: TensorSpec((h * e, w)), n["i"]: TensorSpec((h, w)), n["f"]: TensorSpec((h, w)),
                n["i_bias"]: TensorSpec((h,), init="uniform"), n["f_bias"]: TensorSpec((h,), init="uniform"),
                n["o"]: TensorSpec((w, h * e)), n["norm"]: TensorSpec((h * e,), init="ones")}

    def bind(self, tensors) -> None:
        self._fuse(tensors, ("q", "k", "v", "g", "i", "f"))
        self.i_bias, self.f_bias = tensors[self.names["i_bias"]], tensors[self.names["f_bias"]]

    def state_need(self) -> StateNeed:
        return StateNeed((StateTensor("S", (self.heads, self.dim, self.value_dim), "float32"),
                          StateTensor("n", (self.heads, self.dim), "float32"), StateTensor("m", (self.heads,), "float32")))

    def forward(self, x, batch, cache, state, residual):
        ops = self.rt.ops
        x32 = ops.linear(x, self.proj, out_dtype=torch.float32)
        o = ops.gated_recurrence(x32, self.columns, self.heads, self.dim, self.value_dim, batch, state, mode="exp_gates",
                                 q_scale=self.dim ** -0.5, cap=self.cap, i_bias=self.i_bias, f_bias=self.f_bias)
        return self._finish(o, x32, self.value_dim, residual)

    def parameters_bytes(self) -> int:
        return super().parameters_bytes() + sum(t.numel() * t.element_size() for t in (self.i_bias, self.f_bias))


@register("mixer", "wkv")
class WKV(_RecurrentMixer):
    NAMES = {"r": "r", "k": "k", "v": "v", "g": "g", "w1": "w1", "w2": "w2", "w0": "w0", "u": "u", "o": "o", "norm": "norm",
             "mu_r": "mu.r", "mu_k": "mu.k", "mu_v": "mu.v", "mu_g": "mu.g", "mu_w": "mu.w"}
    BLENDS = ("r", "k", "v", "g", "w")  # the order of the blends; the decay's first step is the fifth product
    STACKED_ROWS = 16  # tokens of a step up to which r, k, v and the gate are one product of stacked blends

    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        if self.value_dim != self.dim:
            raise ValueError(f"wkv heads have keys and values of one size, not {self.dim} / {self.value_dim}")
        # the width of the decay's first step: a configuration may state it; else the checkpoint's tensors say it
        self.rank = int(spec["decay_rank"]) if spec.get("decay_rank") else None
        self.ld = 0
        self.mu = self.weights = self.stacked = self.w2 = self.w0 = self.u = None

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        n = _named(spec, cls.NAMES)
        w, h, d = int(spec["hidden_size"]), int(spec["num_heads"]), int(spec["head_dim"])
        r = int(spec["decay_rank"]) if spec.get("decay_rank") else None
        free = None if r is not None else max(8, min(64, w // 16))
        out = {n[k]: TensorSpec((h * d, w)) for k in ("r", "k", "v", "g")}
        out.update({n[f"mu_{k}"]: TensorSpec((w,), init="uniform") for k in cls.BLENDS})
        out.update({n["w1"]: TensorSpec((r, w), free=free), n["w2"]: TensorSpec((h * d, r), free=free),
                    n["w0"]: TensorSpec((h * d,), init="uniform"),
                    n["u"]: TensorSpec((h, d), init="uniform"), n["norm"]: TensorSpec((h * d,), init="ones"),
                    n["o"]: TensorSpec((w, h * d))})
        return out

    def bind(self, tensors) -> None:
        n = self.names
        parts = [tensors[n[k]] for k in ("r", "k", "v", "g", "w1")]
        if len({t.dtype for t in parts}) != 1:
            raise ValueError(f"{n['r']} and its neighbours are stored in different dtypes")
        # r, k, v and the gate stacked: a step of few tokens multiplies its stacked blends by all of them at once (each
        # blend by every weight: four times the multiply-adds, the weights read once, two launches for eight) and reads
        # each projection off its own block of rows; the single weights are the stacked one's runs of rows, no copies
        self.stacked = torch.cat(parts[:4], dim=0).contiguous()
        rows = parts[0].shape[0]
        self.weights = [self.stacked[i * rows : (i + 1) * rows] for i in range(4)] + [parts[4]]
        dtype = self.weights[0].dtype
        self.rank = self.weights[4].shape[0]
        if tensors[n["w2"]].shape[1] != self.rank:
            raise ValueError(f"{n['w1']} has {self.rank} rows, {n['w2']} {tensors[n['w2']].shape[1]} columns")
        at = 0
        width = self.heads * self.dim
        for k, cols in (("q", width), ("k", width), ("v", width), ("g", width)):  # q: the receptance
            self.columns[k] = at
            at += -(-cols // 4) * 4  # every product's columns start 16-byte aligned
        self.ld = at
        self.mu = torch.stack([tensors[n[f"mu_{k}"]].to(dtype) for k in self.BLENDS]).contiguous()
        self.w2 = tensors[n["w2"]].to(torch.float32).contiguous()  # the decay's second step is a true 32-bit product (widening is exact)
        self.w0 = tensors[n["w0"]]
        self.u = tensors[n["u"]].to(torch.float32).contiguous()
        self.o, self.norm = tensors[n["o"]], tensors[n["norm"]]

    def state_need(self) -> StateNeed:
        return StateNeed((StateTensor("S", (self.heads, self.dim, self.dim), "float32"),
                          StateTensor("shift", (self.hidden,), "float32")))

    def forward(self, x, batch, cache, state, residual):
        ops = self.rt.ops
        c, n, t = self.columns, self.heads * self.dim, x.shape[0]
        blends = ops.token_shift_mix(ops.cast(x, self.mu.dtype), self.mu, state["shift"], batch)
        decay = ops.channel_decay(ops.linear(blends[4], self.weights[4], out_dtype=torch.float32), self.w2, self.w0, log=True)
        if t <= self.STACKED_ROWS and self.stacked.dtype == torch.bfloat16:
            # block j of rows holds every product of blend j; the one that is wanted of it is its j-th run of columns
            all32 = ops.linear(blends[:4].reshape(4 * t, self.hidden), self.stacked, out_dtype=torch.float32)
            ld = 4 * n
            at = {k: j * t * ld + j * n for j, k in enumerate(("q", "k", "v"))}
            gate = all32[3 * t :, 3 * n :]
            o = ops.gated_recurrence(all32[:t], at, self.heads, self.dim, self.dim, batch, state, mode="wkv", channel_decay=decay,
                                     bonus=self.u, rows_below=3 * t)
        else:
            x32 = torch.empty((t, self.ld), dtype=torch.float32, device=x.device)
            for i, (k, w) in enumerate(zip(("q", "k", "v", "g"), self.weights)):
                ops.linear(blends[i], w, out=x32[:, c[k] : c[k] + w.shape[0]])
            gate = x32[:, c["g"] : c["g"] + n]
            o = ops.gated_recurrence(x32, c, self.heads, self.dim, self.dim, batch, state, mode="wkv", channel_decay=decay, bonus=self.u)
        y = ops.group_rmsnorm_gate(o, self.dim, self.norm, gate, self.eps, self.rt.dtype, "silu")
        return ops.linear(y, self.o, accumulate_into=residual, defer=True)

    def parameters_bytes(self) -> int:
        ts = self.weights + [self.mu, self.w2, self.w0, self.u, self.o, self.norm]
        return sum(t.numel() * t.element_size() for t in ts)

    def flops(self, rows) -> int:
        tokens = sum(n for n, _ in rows)
        n = self.heads * self.dim
        rank = self.rank or 0
        linear = 2 * tokens * self.hidden * (4 * n + rank) + 2 * tokens * rank * n + 2 * tokens * n * self.hidden
        return linear + 6 * tokens * self.heads * self.dim * self.dim


@register("mixer", "normed_pair")
class NormedPair(Mixer):
    """Two mixers side by side on the same input: ``coef * (rmsnorm(left(h)) w_left + rmsnorm(right(h)) w_right)`` with
    the norms over the model width. The sub-mixers are any registered mixers (``left`` / ``right``: their ``PartSpec``);
    at most one of them may keep keys and values per token, both may keep state."""

    SIDES = ("left", "right")

    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.hidden = int(spec["hidden_size"])
        self.eps = float(spec["eps"])
        self.coef = float(spec.get("coef", 0.5))
        self.subs = [part_class("mixer", spec[s])(spec[s], rt) for s in self.SIDES]
        self.out_names = [spec.get(f"{s}_norm", f"{s}.out") for s in self.SIDES]
        self.out_weights = None
        if sum(m.kv_need() is not None for m in self.subs) > 1:
            raise NotImplementedError("only one of two mixers side by side may keep keys and values per token")

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        out = {}
        for s in cls.SIDES:
            out.update(part_class("mixer", spec[s]).tensors(spec[s]))
            out[spec.get(f"{s}_norm", f"{s}.out")] = TensorSpec((int(spec["hidden_size"]),), init="ones")
        return out

    @classmethod
    def aliases(cls, spec: PartSpec) -> dict[str, str]:
        out = {}
        for s in cls.SIDES:
            out.update(part_class("mixer", spec[s]).aliases(spec[s]))
        return out

    def bind(self, tensors) -> None:
        for m in self.subs:
            names = list(type(m).tensors(m.spec)) + list(type(m).aliases(m.spec))
            m.bind({n: tensors[n] for n in names})
        self.out_weights = [tensors[n] for n in self.out_names]

    def kv_need(self) -> KVNeed | None:
        return next((n for n in (m.kv_need() for m in self.subs) if n is not None), None)

    def state_need(self) -> StateNeed | None:
        tensors = []
        for side, m in zip(self.SIDES, self.subs):
            need = m.state_need()
            if need is not None:
                tensors += [StateTensor(f"{side}.{t.name}", t.shape, t.dtype) for t in need.tensors]
        return StateNeed(tuple(tensors)) if tensors else None

    def forward(self, x, batch, cache, state, residual):
        ops = self.rt.ops
        streams = []
        for side, m in zip(self.SIDES, self.subs):
            # each mixer adds into a stream of its own, which starts at zero
            own = torch.zeros_like(residual)
            sub_state = {k[len(side) + 1:]: v for k, v in (state or {}).items() if k.startswith(side + ".")}
            pending = m.forward(x, batch, cache if m.kv_need() is not None else None, sub_state or None, own)
            ops.add_pending(own, pending)
            streams.append(own)
        ops.normed_mean_add(residual, streams, self.out_weights, self.eps, self.coef)
        return None

    def parameters_bytes(self) -> int:
        return sum(m.parameters_bytes() for m in self.subs) + sum(w.numel() * w.element_size() for w in self.out_weights)

    def flops(self, rows) -> int:
        return sum(m.flops(rows) for m in self.subs)
