"""Reselorn, whole sequences, no cache, float64 numpy: one function per mechanism. It shares no code with the
product path.

A Reselorn layer norms what a sublayer puts out, not what it reads, and scales it per channel:
``x += ls1 * N1(mixer(x))``, then ``x += ls2 * N2(ff(x))``, with ``N(y) = y / rms(y) * w``. The mixer is grouped-query
attention: a rotation over the first ``rot.dims`` elements of each query and key head (halves paired) whose long
wavelengths are slowed down and whose cosines and sines carry a magnitude; after the rotation queries and keys are
divided by their root mean square per head; a sliding window; a learned sink per head in the softmax's denominator;
and, in layers that say so, values blended with the values the first such layer made of the same token. The
feed-forward is gated (``down(silu(gate x) * up x)``), either one dense layer or a mixture: a router picks ``top`` of
``experts`` small gated layers per token, weighs them by the softmax over the picked logits, and a shared expert is
added for every token. The head is the embedding table.

Notation: T tokens, W width, H heads, G key/value heads, D query/key size, E value size, R rotated elements.
"""

from __future__ import annotations

import math

import numpy as np


# ---------------------------------------------------------------- norms and activations


def unit_rms(x, eps):
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def silu(z):
    return z / (1.0 + np.exp(-z))


# ---------------------------------------------------------------- rotation


def slowed_frequencies(dims, base, scaling):
    """``f_i = base^(-2i/dims)``, ``i < dims/2``, and with ``scaling`` (factor, original, fast, slow) the blend
    ``f_i / factor * r_i + f_i (1 - r_i)``: ``r`` rises from 0 to 1 between the indices at which a wave makes ``fast``
    and ``slow`` turns within ``original`` positions. Returns the frequencies and the magnitude of cos and sin."""
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
    f, mag = slowed_frequencies(R, float(rot["base"]), rot.get("scaling"))
    ang = positions.astype(np.float64)[:, None] * f  # [T, R/2]
    cos, sin = (np.cos(ang) * mag)[:, None, :], (np.sin(ang) * mag)[:, None, :]
    out = x.copy()
    a, b = x[..., : R // 2], x[..., R // 2 : R]
    out[..., : R // 2] = a * cos - b * sin
    out[..., R // 2 : R] = b * cos + a * sin
    return out


# ---------------------------------------------------------------- softmax over visible keys


def sink_softmax(scores, visible, sink):
    """``scores [T, T]``, ``visible`` boolean of the same shape; ``exp(sink)`` joins the denominator once, with
    neither key nor value."""
    s = np.where(visible, scores, -np.inf)
    m = np.maximum(s.max(axis=-1, keepdims=True), sink)
    e = np.where(visible, np.exp(s - m), 0.0)
    return e / (e.sum(axis=-1, keepdims=True) + np.exp(sink - m))


def sliding(T, size):
    i = np.arange(T)
    d = i[:, None] - i[None, :]
    return (d >= 0) & ((d < size) if size else True)


# ---------------------------------------------------------------- mixer


def values_of(h, w, m):
    """The layer's own values ``[T, G, E]``, before any blend."""
    return (h @ w["v"].T).reshape(h.shape[0], m["kv_heads"], m["vdim"])


def blend_values(v, v_first, lam):
    return (1.0 - lam) * v + lam * v_first


def attention(h, w, m, eps, positions, v):
    """``v``: the values the layer attends over (blended already where the layer blends)."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).reshape(T, H, D)
    k = (h @ w["k"].T).reshape(T, G, D)
    if m.get("rot"):
        q, k = rotate_halves(q, positions, m["rot"]), rotate_halves(k, positions, m["rot"])
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    seen = sliding(T, m["mask"]["size"] if m.get("mask") else 0)
    out = np.zeros((T, H, E))
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"]
        out[:, head] = sink_softmax(s, seen, float(w["sink"][head])) @ v[:, g]
    return out.reshape(T, H * E) @ w["o"].T


# ---------------------------------------------------------------- feed-forwards


def gated_ff(h, w):
    return (silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def route(h, w, top):
    """Per token the ``top`` experts with the largest router logits, largest first, and the softmax over those logits."""
    z = h @ w["router"].T + w["router.b"]
    chosen = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    zc = np.take_along_axis(z, chosen, axis=-1)
    e = np.exp(zc - zc.max(axis=-1, keepdims=True))
    return chosen, e / e.sum(axis=-1, keepdims=True)


def mixture_ff(h, w, mlp):
    chosen, weight = route(h, w, mlp["router"]["top"])
    out = np.zeros((h.shape[0], w["e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, p in zip(chosen[t], weight[t]):
            out[t] += p * gated_ff(h[t : t + 1], _sub(w, f"e{e}."))[0]
    if mlp.get("shared"):
        out += gated_ff(h, _sub(w, "shared."))
    return out


# ---------------------------------------------------------------- the model


def _sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, return_layers=False):
    """Logits ``[T, vocab]`` of one sequence (and, asked for, the stream after every layer ``[layers, T, W]``)."""
    eps = cfg["norm"]["eps"]
    tokens = np.asarray(tokens)
    positions = np.arange(len(tokens))
    x = weights["embed"][tokens].astype(np.float64)
    v_first, after = None, []
    for i, layer in enumerate(cfg["layers"]):
        if layer["type"] != "attention":
            raise ValueError(f"layer {i}: unknown mixer {layer['type']!r}")
        w, m = _sub(weights, f"l{i}.mix."), layer["mixer"]
        v = values_of(x, w, m)
        if m.get("v_mix"):
            if v_first is None:
                v_first = v
            else:
                v = blend_values(v, v_first, float(w["vmix"]))
        y = attention(x, w, m, eps, positions, v)
        x = x + rms_norm(y, weights[f"l{i}.norm1"], eps) * weights[f"l{i}.ls1"]
        mlp = layer.get("mlp")
        if mlp:
            wf = _sub(weights, f"l{i}.mlp.")
            y = gated_ff(x, wf) if mlp["kind"] == "dense" else mixture_ff(x, wf, mlp)
            x = x + rms_norm(y, weights[f"l{i}.norm2"], eps) * weights[f"l{i}.ls2"]
        after.append(x.copy())
    logits = rms_norm(x, weights["final.norm"], eps) @ weights["embed"].T
    return (logits, np.stack(after)) if return_layers else logits


def greedy(cfg, weights, prompt, new_tokens):
    """The ``new_tokens`` tokens that greedy decoding appends to ``prompt`` (the whole sequence is run again each time)."""
    toks = list(prompt)
    for _ in range(new_tokens):
        toks.append(int(np.argmax(forward(cfg, weights, toks)[-1])))
    return toks[len(prompt):]
