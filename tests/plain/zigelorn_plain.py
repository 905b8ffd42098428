"""Zigelorn, whole sequences, no cache, float64 numpy: one function per mechanism. It shares no code with the
product path.

A Zigelorn layer norms what a sublayer reads and what it puts out: ``x += N1b(mixer(N1(x)))``, then
``x += N2b(ff(N2(x)))``, with ``N(y) = y / rms(y) * (1 + w)``. Three mixers:

* ``attention``: grouped-query heads whose values are the keys as projected (no value projection); biases on both
  projections; one RMS norm over a token's whole query projection and one over its whole key projection; a rotation
  over the first ``rot.dims`` elements of each head (halves paired) whose long wavelengths may be slowed down; a
  sliding window; a sigmoid gate per head read off the mixer's input.
* ``retention``: linear attention with a constant decay per head, ``S_t = decay S_(t-1) + k_t v_t^T``,
  ``o_t = S_t^T q_t``, rotated q and k, each head's output divided by its root mean square, a SiLU gate.
* ``wkv``: every projection reads its own blend of the token's input and the previous token's; a decay per key
  channel and token, ``exp(-exp(.))`` of a small two-step projection; ``o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t``,
  then ``S_t = diag(w_t) S_(t-1) + k_t v_t^T``; a norm per head, a weight, a SiLU gate.

Feed-forwards: ``down(gelu_tanh(up x))``, or a mixture of such layers with a squared ReLU: the router's softmax over
real and identity experts, a correction that only the choice sees, groups of neighbours of which the best are kept,
weights that are the chosen experts' softmax values as they stand. The head is the embedding table.

Notation: T tokens, W width, H heads, G key/value heads, D query/key size, E value size, R rotated elements.
"""

from __future__ import annotations

import math

import numpy as np


# ---------------------------------------------------------------- rounding, for error estimates


def no_rounding(a):
    return a


def to_bfloat16(a):
    """``a`` rounded to the nearest bfloat16 (ties to even), as float64: what a 16-bit product is fed."""
    bits = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    bits = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
    return bits.astype(np.uint32).view(np.float32).astype(np.float64).reshape(np.shape(a))


# What every matrix product's input goes through. ``forward(..., rounding=to_bfloat16)`` rounds them as a 16-bit engine
# must (norm outputs, blends, what the output and down projections read), and nothing else: the difference to the exact
# result is a sample of the error that rounding alone causes at each position.
_round = no_rounding


# ---------------------------------------------------------------- norms and activations


def unit_rms(x, eps):
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def one_plus_norm(x, w, eps):
    return unit_rms(x, eps) * (1.0 + w)


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def relu_squared(z):
    return np.maximum(z, 0.0) ** 2


# ---------------------------------------------------------------- rotation


def frequencies(dims, base, scaling):
    """``f_i = base^(-2i/dims)``, ``i < dims/2``; with ``scaling`` (factor, original, fast, slow) the blend
    ``f_i / factor * r_i + f_i (1 - r_i)``, ``r`` rising from 0 to 1 between the indices at which a wave makes ``fast``
    and ``slow`` turns within ``original`` positions. Returns the frequencies and what cos and sin are multiplied by."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def index_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(index_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(index_of(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_halves(x, positions, rot):
    """Turns the pairs (i, i + R/2), i < R/2, of the last axis of ``x [T, heads, >= R]``; what lies behind R passes."""
    R = rot["dims"]
    f, mag = frequencies(R, float(rot["base"]), rot.get("scaling"))
    ang = positions.astype(np.float64)[:, None] * f
    cos, sin = (np.cos(ang) * mag)[:, None, :], (np.sin(ang) * mag)[:, None, :]
    out = x.copy()
    a, b = x[..., : R // 2], x[..., R // 2 : R]
    out[..., : R // 2] = a * cos - b * sin
    out[..., R // 2 : R] = b * cos + a * sin
    return out


# ---------------------------------------------------------------- mixers


def sliding(T, size):
    i = np.arange(T)
    d = i[:, None] - i[None, :]
    return (d >= 0) & ((d < size) if size else True)


def softmax_over(scores, visible):
    s = np.where(visible, scores, -np.inf)
    e = np.where(visible, np.exp(s - s.max(axis=-1, keepdims=True)), 0.0)
    return e / e.sum(axis=-1, keepdims=True)


def attention(h, w, m, eps, positions):
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = h @ w["q"].T + w["q.b"]
    k = h @ w["k"].T + w["k.b"]
    v = k.reshape(T, G, D)  # the values are the keys as projected
    q = (unit_rms(q, eps) * w["q.norm"]).reshape(T, H, D)
    k = (unit_rms(k, eps) * w["k.norm"]).reshape(T, G, D)
    if m.get("rot"):
        q, k = rotate_halves(q, positions, m["rot"]), rotate_halves(k, positions, m["rot"])
    seen = sliding(T, m["mask"]["size"] if m.get("mask") else 0)
    gate = sigmoid(h @ w["g"].T)  # [T, H]
    out = np.zeros((T, H, D))
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"]
        out[:, head] = (softmax_over(s, seen) @ v[:, g]) * gate[:, head : head + 1]
    return _round(out.reshape(T, H * D)) @ w["o"].T


def retention(h, w, m, eps, positions):
    T = h.shape[0]
    H, D, E = m["heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).reshape(T, H, D)
    k = (h @ w["k"].T).reshape(T, H, D)
    v = (h @ w["v"].T).reshape(T, H, E)
    if m.get("rot"):
        q, k = rotate_halves(q, positions, m["rot"]), rotate_halves(k, positions, m["rot"])
    k = k * D**-0.5
    out = np.zeros((T, H, E))
    for head in range(H):
        S = np.zeros((D, E))
        for t in range(T):
            S = float(m["decay"][head]) * S + np.outer(k[t, head], v[t, head])
            out[t, head] = S.T @ q[t, head]
    out = unit_rms(out, eps).reshape(T, H * E) * silu(h @ w["g"].T)
    return _round(out) @ w["o"].T


def shifted(h):
    """The previous token's row for every token; zeros for the first."""
    return np.concatenate([np.zeros_like(h[:1]), h[:-1]], axis=0)


def wkv(h, w, m, eps):
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    back = shifted(h) - h
    mix = {s: _round(h + back * w[f"mu.{s}"]) for s in "rkvgw"}
    r = (mix["r"] @ w["r"].T).reshape(T, H, D)
    k = (mix["k"] @ w["k"].T).reshape(T, H, D)
    v = (mix["v"] @ w["v"].T).reshape(T, H, D)
    gate = silu(mix["g"] @ w["g"].T)
    decay = np.exp(-np.exp(np.tanh(mix["w"] @ w["w1"].T) @ w["w2"].T + w["w0"])).reshape(T, H, D)
    out = np.zeros((T, H, D))
    for head in range(H):
        S = np.zeros((D, D))
        for t in range(T):
            kv = np.outer(k[t, head], v[t, head])
            out[t, head] = (S + w["u"][head][:, None] * kv).T @ r[t, head]
            S = decay[t, head][:, None] * S + kv
    out = unit_rms(out, eps).reshape(T, H * D) * w["norm"] * gate
    return _round(out) @ w["o"].T


# ---------------------------------------------------------------- feed-forwards


def dense_ff(h, w):
    return _round(gelu_tanh(h @ w["up"].T)) @ w["down"].T


def route(h, w, router):
    """Per token the chosen experts, largest choice score first, and their weights. Numbers from ``experts`` on are
    identity experts."""
    z = h @ w["router"].T
    e = np.exp(z - z.max(axis=-1, keepdims=True))
    s = e / e.sum(axis=-1, keepdims=True)
    choice = s + w["correction"]
    groups = router.get("groups")
    if groups:
        n = choice.shape[-1] // groups["count"]
        best = choice.reshape(-1, groups["count"], n).max(axis=-1)
        kept = np.argsort(-best, axis=-1, kind="stable")[:, : groups["keep"]]
        allowed = np.zeros(best.shape, dtype=bool)
        np.put_along_axis(allowed, kept, True, axis=-1)
        choice = np.where(np.repeat(allowed, n, axis=-1), choice, -np.inf)
    chosen = np.argsort(-choice, axis=-1, kind="stable")[:, : router["top"]]
    return chosen, np.take_along_axis(s, chosen, axis=-1)


def mixture_ff(h, w, mlp):
    router = mlp["router"]
    chosen, weight = route(h, w, router)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, p in zip(chosen[t], weight[t]):
            if e >= router["experts"]:
                out[t] += p * h[t]
            else:
                out[t] += p * (_round(relu_squared(h[t] @ w[f"e{e}.up"].T)) @ w[f"e{e}.down"].T)
    return out


# ---------------------------------------------------------------- the model


def weights_layer(cfg, i):
    """The layer whose tensors layer ``i`` runs: itself, or the end of its chain of ``weights_of``."""
    while cfg["layers"][i].get("weights_of") is not None:
        i = cfg["layers"][i]["weights_of"]
    return i


def _sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, return_layers=False, watch=None, rounding=None):
    """Logits ``[T, vocab]`` of one sequence (and, asked for, the stream after every layer ``[layers, T, W]``).
    ``watch(i, x)`` is shown the stream that layer ``i``'s feed-forward norm reads. ``rounding``: see ``_round``."""
    global _round
    before, _round = _round, rounding or no_rounding
    try:
        return _forward(cfg, weights, tokens, return_layers, watch)
    finally:
        _round = before


def _forward(cfg, weights, tokens, return_layers, watch):
    eps = cfg["norm"]["eps"]
    tokens = np.asarray(tokens)
    positions = np.arange(len(tokens))
    x = weights["embed"][tokens].astype(np.float64)
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{weights_layer(cfg, i)}."
        w, m = _sub(weights, p + "mix."), layer["mixer"]
        h = _round(one_plus_norm(x, weights[p + "norm1"], eps))
        if layer["type"] == "attention":
            y = attention(h, w, m, eps, positions)
        elif layer["type"] == "retention":
            y = retention(h, w, m, eps, positions)
        elif layer["type"] == "wkv":
            y = wkv(h, w, m, eps)
        else:
            raise ValueError(f"layer {i}: unknown mixer {layer['type']!r}")
        x = x + one_plus_norm(y, weights[p + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp:
            wf = _sub(weights, p + "mlp.")
            if watch is not None:
                watch(i, x)
            h = _round(one_plus_norm(x, weights[p + "norm2"], eps))
            y = dense_ff(h, wf) if mlp["kind"] == "dense" else mixture_ff(h, wf, mlp)
            x = x + one_plus_norm(y, weights[p + "norm2b"], eps)
        after.append(x.copy())
    logits = _round(one_plus_norm(x, weights["final.norm"], eps)) @ weights["embed"].T
    return (logits, np.stack(after)) if return_layers else logits


def greedy(cfg, weights, prompt, new_tokens):
    """The ``new_tokens`` tokens that greedy decoding appends to ``prompt`` (the whole sequence is run again each time)."""
    toks = list(prompt)
    for _ in range(new_tokens):
        toks.append(int(np.argmax(forward(cfg, weights, toks)[-1])))
    return toks[len(prompt):]
