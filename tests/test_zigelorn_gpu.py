"""Zigelorn on the GPU against the plain implementation (``tests/plain/zigelorn_plain.py``): every mechanism alone on
inputs made so that a fault shows, then whole models with random weights under every kind of schedule: whole prompts,
token-by-token decoding, portions down to two tokens, batches of unequal requests, pages and slots that are given back
and used again, long decoding, greedy generation through the engine and its scheduler, and the trace replay tool."""

from __future__ import annotations

import copy
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from plain import zigelorn_plain as Z
from plain.model_folder import read_model_folder
from tolerances import check_logits_against_rounding
from tolerances import check_logits_by_position as check_logits
from zigelorn_models import ZIGELORN, make_folder, tokens_for

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
PAGE = 16


def ops():
    from miniserve_amd.kernels import ops as o

    o.library()
    return o


def dev(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV).contiguous()


def rounded(a, dtype):
    """What a kernel is given when ``a`` is stored in ``dtype``."""
    return dev(a, dtype).float().cpu().numpy().astype(np.float64)


def close(got, want, dtype, what="", tol=None):
    got = got.float().cpu().numpy().astype(np.float64)
    scale = max(float(np.abs(want).max()), 1e-30)
    tol = tol or (2e-5 if dtype == torch.float32 else 1.2e-2)
    worst = float(np.abs(got - want).max())
    assert worst <= tol * scale, f"{what}: max |diff| {worst:.3e} > {tol * scale:.3e}"


def step_batch(lens, starts, slots=None):
    """What the kernels read of a step: rows of ``lens`` new tokens behind ``starts`` cached ones."""
    pos = np.concatenate([np.arange(s, s + n) for n, s in zip(lens, starts)])
    row = np.concatenate([np.full(n, i) for i, n in enumerate(lens)])
    flat = np.arange(int(sum(lens)))
    single = np.concatenate([np.full(n, n == 1) for n in lens])
    n_dec = int(single.sum())
    mixed = 0 < n_dec < len(flat)
    b = SimpleNamespace(num_rows=len(lens), num_tokens=int(sum(lens)), positions=dev(pos, torch.int32), token_row=dev(row, torch.int32),
                        row_start=dev(np.concatenate(([0], np.cumsum(lens))), torch.int32), starts=dev(starts, torch.int32),
                        state_slots=dev(list(range(len(lens))) if slots is None else slots, torch.int32),
                        num_decode_tokens=n_dec, decode_tokens=dev(flat[single], torch.int32) if mixed else None,
                        prefill_tokens=dev(flat[~single], torch.int32) if mixed else None,
                        max_kv_len=max(s + n for n, s in zip(lens, starts)), row_lens=list(lens), row_starts_host=list(starts), memo={})
    b.is_decode = n_dec == len(flat)
    return b


def rope_for(o, pos, rot):
    if rot is None:
        return None
    f, mag = Z.frequencies(rot["dims"], float(rot["base"]), rot.get("scaling"))
    return o.rope_table(dev(pos, torch.int32), dev(f.astype(np.float32)), mag)


CUTS = ([400], [150] + [1] * 250, [2, 3, 64, 5, 2, 31, 1, 1, 190, 1, 100])


# ---------------------------------------------------------------- mechanisms alone


def test_a_product_into_the_columns_of_a_wider_matrix():
    """Several products share one float32 matrix; each writes its own run of columns and nothing else."""
    o = ops()
    rng = np.random.default_rng(0)
    for dtype in (torch.float32, torch.bfloat16):
        for m in (1, 9, 70, 300):
            x, w = rng.normal(size=(m, 96)), rng.normal(size=(40, 96))
            big = torch.full((m, 132), 7.0, dtype=torch.float32, device=DEV)
            o.linear(dev(x, dtype), dev(w, dtype), out=big[:, 44:84])
            close(big[:, 44:84], rounded(x, dtype) @ rounded(w, dtype).T, torch.float32, f"{m} rows", 3e-5)
            assert (big[:, :44] == 7).all() and (big[:, 84:] == 7).all()
            with pytest.raises(ValueError):
                o.linear(dev(x, dtype), dev(w, dtype), out=big[:, 43:83])  # rows that do not start 16-byte aligned


def plain_prepare(x, bias, pos, hq, hk, d, rot, qw, kw, eps):
    """Queries ``[T, hq, d]``, keys ``[T, hk, d]`` and values ``[T, hk, d]`` from projection rows ``[T, (hq + hk) d]``."""
    T = x.shape[0]
    x = x + bias
    q, k = x[:, : hq * d], x[:, hq * d :]
    v = k.reshape(T, hk, d)
    q = (Z.unit_rms(q, eps) * qw).reshape(T, hq, d)
    k = (Z.unit_rms(k, eps) * kw).reshape(T, hk, d)
    if rot is not None:
        q, k = Z.rotate_halves(q, pos, rot), Z.rotate_halves(k, pos, rot)
    return q, k, v


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hq,hk,d,rot", [
    (4, 2, 16, {"dims": 8, "base": 500.0, "scaling": {"factor": 4.0, "original": 32, "fast": 4.0, "slow": 0.5}}),
    (3, 1, 10, {"dims": 6, "base": 300.0}), (2, 2, 14, {"dims": 14, "base": 300.0}), (8, 2, 64, None),
    (1, 1, 300, {"dims": 2, "base": 10.0}),
])
def test_norm_over_the_projection_with_biases_and_values_that_are_the_keys(hq, hk, d, rot, dtype):
    """One norm over all of a token's queries and one over all of its keys, the biases added first, a part of every head
    turned, and the keys as projected (bias in, norm and rotation not) stored as the values. One token's queries are tiny
    against eps, so eps under the root shows; the gate's columns lie behind the keys and are not touched."""
    o = ops()
    rng = np.random.default_rng(hq * d)
    T, eps = 37, 1e-3
    x = rng.normal(size=(T, (hq + hk) * d + hq))
    bias = rng.normal(size=(hq + hk) * d) * 0.5
    pos = np.concatenate([np.arange(100, 100 + T - 5), np.arange(5)])
    qw, kw = rng.normal(size=hq * d) + 1, rng.normal(size=hk * d) + 1
    wdt = dtype
    br, qwr, kwr = rounded(bias, wdt), rounded(qw, wdt), rounded(kw, wdt)
    x[3, : hq * d] = rng.normal(size=hq * d) * 1e-3 - br[: hq * d]  # tiny once the bias is in
    q, k, v = plain_prepare(x[:, : (hq + hk) * d], br, pos, hq, hk, d, rot, qwr, kwr, eps)
    slots = rng.permutation(4 * PAGE)[:T]
    kc = torch.zeros((5, hk, PAGE, d), dtype=dtype, device=DEV)
    vc = torch.zeros((5, hk, d, PAGE), dtype=dtype, device=DEV)
    got = o.qkv_norm_rope_store(dev(x), dev(slots, torch.int32), dev(qw, wdt), dev(kw, wdt), eps, rope_for(o, pos, rot), kc, vc, hq, hk, d, d,
                                dtype, "halves", dev(bias, wdt), True, hq)
    tol = 2e-5 if dtype == torch.float32 else 5e-3
    close(got, q.reshape(T, -1), dtype, "queries", tol)
    at = dev(slots, torch.int64)
    close(kc.permute(0, 2, 1, 3).reshape(-1, hk, d)[at], k, dtype, "keys", tol)
    close(vc.permute(0, 3, 1, 2).reshape(-1, hk, d)[at], v, dtype, "values", tol)
    assert np.abs(v - k).max() > 0.1  # the values are not the finished keys
    with pytest.raises(ValueError):
        o.qkv_norm_rope_store(dev(x), None, dev(qw, wdt), dev(kw, wdt), eps, None, None, None, hq, hk, d, d + 1, dtype, "halves", None, True, hq)


def plain_attention(q, k, v, scale, size, gate):
    T, H, _ = q.shape
    per = H // k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for a in range(H):
        s = (q[:, a] @ k[:, a // per].T) * scale
        out[:, a] = (Z.softmax_over(s, Z.sliding(T, size)) @ v[:, a // per]) * gate[:, a : a + 1]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hq,hk,d,size,dims", [(4, 2, 32, 37, 16), (3, 1, 10, 16, 6), (8, 2, 64, 100, 32), (6, 3, 48, 0, 48),
                                               (4, 1, 128, 70, 64), (4, 4, 40, 17, 0), (4, 2, 32, 1, 16), (2, 1, 64, 2, 32),
                                               (2, 2, 24, 33, 24)])
def test_gated_attention_whose_values_are_its_keys(hq, hk, d, size, dims, dtype):
    """Projection rows through bias, norm, rotation and store into pages, then attention inside a window and the gate per
    head, in cuts of every kind. For the last query of every group's first head, the key just inside the window and the
    key just outside it are made to meet that query (the outer one large among the values), and a key far back likewise
    where every key is seen: a window one token off, a lost page or a wrong head pairing shows."""
    o = ops()
    rng = np.random.default_rng(hq * d + size)
    T, scale, eps = 400, 6.0 / np.sqrt(d), 1e-5
    rot = {"dims": dims, "base": 1000.0, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}} if dims else None
    per = hq // hk
    nq, nk = hq * d, hk * d
    x = rng.normal(size=(T, nq + nk + hq))
    bias = rng.normal(size=nq + nk) * 0.3
    qw, kw = np.ones(nq), np.ones(nk)
    pos = np.arange(T)
    # plant keys: the finished key at `at` equals the finished query of the last token's head a, turned back to `at`
    q0, _, _ = plain_prepare(x[:, : nq + nk], bias, pos, hq, hk, d, None, qw, kw, eps)  # normed, not turned
    k_rms = np.sqrt(((x[:, nq : nq + nk] + bias[nq:]) ** 2).mean(-1) + eps)
    for g in range(hk):
        a = g * per
        inner, outer = (T - size, T - size - 1) if size else (3 + 5 * g, None)
        for at in (inner, outer):
            if at is None or at < 0 or at >= T - 1:
                continue
            # a key row whose normed form is the query's normed form (same direction; the norm takes the length)
            x[at, nq + g * d : nq + (g + 1) * d] = q0[T - 1, a] * (3.0 if at == inner else 9.0) * k_rms[at] - bias[nq + g * d : nq + (g + 1) * d]  # (the outer one three times as long: so is its value)
    q, k, v = plain_prepare(x[:, : nq + nk], bias, pos, hq, hk, d, rot, qw, kw, eps)
    gate = Z.sigmoid(x[:, nq + nk :])
    qr, kr, vr = rounded(q, dtype), rounded(k, dtype), rounded(v, dtype)
    want = plain_attention(qr, kr, vr, scale, size, gate)
    if size > 1 and dims == 0:  # (a turned key meets the query at its own place only where nothing is turned)
        seen = plain_attention(qr, kr, vr, scale, size + 1, gate)
        assert np.abs(seen - want)[T - 1].max() > 0.05 * np.abs(want[T - 1]).max()
        lost = plain_attention(qr, kr, vr, scale, size - 1, gate)
        assert np.abs(lost - want)[T - 1].max() > 0.05 * np.abs(want[T - 1]).max()
    pages = [int(p) for p in rng.permutation(30)[: -(-T // PAGE)]]
    kc = torch.zeros((31, hk, PAGE, d), dtype=dtype, device=DEV)
    vc = torch.zeros((31, hk, d, PAGE), dtype=dtype, device=DEV)
    table = dev([pages + [0] * (-len(pages) % 4)], torch.int32)
    tol = 2e-5 if dtype == torch.float32 else 8e-3
    for cuts in CUTS:
        kc.zero_(); vc.zero_()
        got, at = [], 0
        for n in cuts:
            n = min(n, T - at)
            if n <= 0:
                break
            b = step_batch([n], [at])
            slots = [pages[p // PAGE] * PAGE + p % PAGE for p in range(at, at + n)]
            xs = dev(x[at : at + n])
            qs = o.qkv_norm_rope_store(xs, dev(slots, torch.int32), dev(qw), dev(kw), eps, rope_for(o, np.arange(at, at + n), rot), kc, vc,
                                       hq, hk, d, d, dtype, "halves", dev(bias), True, hq)
            out = o.paged_attention(qs, kc, vc, table, b, hq, hk, d, scale, size, d, 0, True)
            got.append(o.head_gate_(out, xs, nq + nk, hq))
            at += n
        close(torch.cat(got), want.reshape(T, -1), dtype, f"cuts {cuts[:3]}", tol)
    if size:  # the last tokens again, with every page before the window gone
        first_live = (T - 20 - size + 1) // PAGE
        gone = [-1 if i < first_live else p for i, p in enumerate(pages)]
        b = step_batch([20], [T - 20])
        out = o.paged_attention(dev(q.reshape(T, -1), dtype)[T - 20 :].contiguous(), kc, vc, dev([gone + [0] * (-len(gone) % 4)], torch.int32),
                                b, hq, hk, d, scale, size, d, 0, True)
        got = o.head_gate_(out, dev(x[T - 20 :]), nq + nk, hq)
        close(got, want.reshape(T, -1)[T - 20 :], dtype, "pages before the window given away", tol)


@pytest.mark.parametrize("heads,dim,rot,scale", [(3, 12, {"dims": 12, "base": 50.0}, 12 ** -0.5), (2, 16, {"dims": 4, "base": 300.0}, 1.0),
                                                 (5, 6, None, 0.37), (1, 256, {"dims": 64, "base": 1e4, "scaling": {"factor": 8.0, "original": 64,
                                                                                                                     "fast": 16.0, "slow": 1.0}}, 0.0625)])
def test_rotation_of_float32_columns_in_place(heads, dim, rot, scale):
    o = ops()
    rng = np.random.default_rng(heads * dim)
    T = 45
    x = rng.normal(size=(T, 7 + heads * dim + 5))
    pos = np.concatenate([np.arange(20, 20 + T - 3), np.arange(3)])  # (an angle is a float32 product: small places keep it sharp)
    want = x.copy()
    part = x[:, 7 : 7 + heads * dim].reshape(T, heads, dim)
    want[:, 7 : 7 + heads * dim] = ((Z.rotate_halves(part, pos, rot) if rot else part) * scale).reshape(T, -1)
    got = o.rotate_columns_(dev(x), 7, heads, dim, rope_for(o, pos, rot), "halves", scale)
    close(got, want, torch.float32, tol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_blends_with_the_previous_token_and_the_carried_row(dtype):
    """Every cut of two sequences gives the blends of the whole: the previous token comes from the step, from the slot, or
    is zero at a sequence's start; a slot that another request used before does not leak into a new one."""
    o = ops()
    rng = np.random.default_rng(3)
    W, n = 70, 5
    mu = rng.random(size=(n, W))
    seqs = [rng.normal(size=(60, W)), rng.normal(size=(33, W))]
    mr = rounded(mu, dtype)
    want = [rounded(h, dtype)[None] + (Z.shifted(rounded(h, dtype)) - rounded(h, dtype))[None] * mr[:, None, :] for h in seqs]
    carry = torch.full((4, W), 9.0, dtype=torch.float32, device=DEV)  # slots full of another request's rows
    got = [[], []]
    at = [0, 0]
    for lens in ([1, 5], [20, 1], [2, 1], [1, 26], [36, 0]):
        rows = [(i, k) for i, k in enumerate(lens) if k]
        b = step_batch([k for _, k in rows], [at[i] for i, _ in rows], [3 if i == 0 else 1 for i, _ in rows])
        h = np.concatenate([seqs[i][at[i] : at[i] + k] for i, k in rows])
        out = o.token_shift_mix(dev(h, dtype), dev(mu, dtype), carry, b)
        off = 0
        for i, k in rows:
            got[i].append(out[:, off : off + k])
            off += k
            at[i] += k
    for i in range(2):
        close(torch.cat(got[i], dim=1), want[i], dtype, f"sequence {i}", 2e-6 if dtype == torch.float32 else 8e-3)
    assert torch.equal(carry[3], dev(seqs[0][-1], dtype).float()) and (carry[0] == 9).all()


@pytest.mark.parametrize("channels,rank", [(48, 5), (30, 1), (512, 64), (100, 1024)])
def test_decay_per_channel(channels, rank):
    o = ops()
    rng = np.random.default_rng(channels)
    for T in (1, 8, 21, 300):
        a = rng.normal(size=(T, rank))
        w2, w0 = rng.normal(size=(channels, rank)) / np.sqrt(rank), rng.normal(size=channels) - 1.0
        want = np.exp(-np.exp(np.tanh(a) @ w2.T + w0))
        close(o.channel_decay(dev(a), dev(w2), dev(w0)), want, torch.float32, tol=2e-5)
        close(o.channel_decay(dev(a), dev(w2), dev(w0), log=True), np.log(want), torch.float32, tol=2e-5)
        w0b = rounded(w0, torch.bfloat16)
        close(o.channel_decay(dev(a), dev(w2), dev(w0, torch.bfloat16)), np.exp(-np.exp(np.tanh(a) @ w2.T + w0b)), torch.float32, tol=2e-5)
    # a decay of nothing: its logarithm stays a number, so that sums and differences of such logarithms do
    huge = o.channel_decay(dev(np.zeros((2, rank))), dev(np.zeros((channels, rank))), dev(np.full(channels, 200.0)), log=True)
    assert (huge == -200).all()
    assert not o.channel_decay(dev(np.zeros((2, rank))), dev(np.zeros((channels, rank))), dev(np.full(channels, 200.0))).any()


def plain_wkv(r, k, v, w, u):
    """``r, k, v, w [T, H, D]``, ``u [H, D]``: the outputs ``[T, H, D]`` and the last state ``[H, D, D]``."""
    T, H, D = r.shape
    out, S = np.zeros((T, H, D)), np.zeros((H, D, D))
    for t in range(T):
        for h in range(H):
            kv = np.outer(k[t, h], v[t, h])
            out[t, h] = (S[h] + u[h][:, None] * kv).T @ r[t, h]
            S[h] = w[t, h][:, None] * S[h] + kv
    return out, S


@pytest.mark.parametrize("heads,dim", [(3, 10), (2, 64), (1, 8), (4, 32), (1, 200)])
def test_recurrence_with_a_decay_per_channel_and_a_bonus(heads, dim):
    """Two sequences in cuts of every kind against the loop over tokens. One channel hardly decays and an early token is
    large there, so a token far back is most of a late output; a slot that held another request's state starts a new
    request from zero."""
    o = ops()
    rng = np.random.default_rng(heads * dim)
    n = heads * dim
    lens = [180, 47]
    seqs = []
    for T in lens:
        r, k, v = (rng.normal(size=(T, heads, dim)) for _ in range(3))
        w = np.exp(-np.exp(rng.normal(size=(T, heads, dim)) - 1.5))
        w[:, :, 0] = 0.9995
        w[:, :, 1] = 0.0  # a channel that keeps nothing (its logarithm arrives as -200)
        w[5::7, :, 2] = 0.0  # ... and one that forgets everything now and then
        k[2, :, 0] = 30.0
        seqs.append((r, k, v, w))
    u = rng.normal(size=(heads, dim)) + 0.5
    want = [plain_wkv(*s, u) for s in seqs]
    far = plain_wkv(seqs[0][0], np.where(np.arange(lens[0])[:, None, None] == 2, 0.0, seqs[0][1]), seqs[0][2], seqs[0][3], u)[0]
    assert np.abs(far - want[0][0])[-1].max() > 0.3 * np.abs(want[0][0][-1]).max()  # the far token matters at the end
    cols = {"q": 4, "k": 4 + n, "v": 4 + 2 * n}
    for steps in ([[180, 47]], [[100, 0], [1, 1], [1, 0]] + [[1, 1]] * 30 + [[48, 15], [0, 1]], [[2, 3], [3, 2], [17, 1], [64, 40], [94, 1]]):
        S = torch.full((4, heads, dim, dim), 5.0, dtype=torch.float32, device=DEV)
        got, at = [[], []], [0, 0]
        for step in steps:
            rows = [(i, min(c, lens[i] - at[i])) for i, c in enumerate(step)]
            rows = [(i, c) for i, c in rows if c > 0]
            if not rows:
                continue
            b = step_batch([c for _, c in rows], [at[i] for i, _ in rows], [2 if i == 0 else 0 for i, _ in rows])
            x = np.zeros((b.num_tokens, 4 + 3 * n + 3))
            wd = np.zeros((b.num_tokens, n))
            off = 0
            for i, c in rows:
                r, k, v, w = (a[at[i] : at[i] + c].reshape(c, n) for a in seqs[i])
                x[off : off + c, 4 : 4 + 3 * n] = np.concatenate([r, k, v], axis=1)
                wd[off : off + c] = w
                off += c
            out = o.gated_recurrence(dev(x), cols, heads, dim, dim, b, {"S": S}, mode="wkv", channel_decay=dev(np.where(wd > 0, np.log(np.maximum(wd, 1e-300)), -200.0)), bonus=dev(u))
            off = 0
            for i, c in rows:
                got[i].append(out[off : off + c])
                off += c
                at[i] += c
        for i in range(2):
            if at[i] == lens[i]:
                close(torch.cat(got[i]), want[i][0].reshape(lens[i], n), torch.float32, f"sequence {i}", 3e-5)
        close(S[2], want[0][1], torch.float32, "the state that is kept", 3e-5)


@pytest.mark.parametrize("heads,dim,vdim,decay,rot", [(2, 16, 24, [0.9, 0.99], {"dims": 16, "base": 100.0}), (5, 6, 14, [0.7, 0.9, 0.95, 0.99, 0.999], {"dims": 4, "base": 300.0}),
                                                      (2, 128, 64, [0.97, 0.9995], {"dims": 64, "base": 1000.0}), (2, 4, 8, [0.0, 1.0], None)])
def test_retention_in_cuts(heads, dim, vdim, decay, rot):
    """Rotation, the keys' scale, the recurrence with a decay per head (token by token and in chunks), the norm per head
    without a weight and the SiLU gate, in cuts of every kind against the loop over tokens."""
    o = ops()
    rng = np.random.default_rng(heads * dim)
    T, eps = 230, 1e-5
    nq, nv = heads * dim, heads * vdim
    x = rng.normal(size=(T, 2 * nq + 2 * nv))
    x[5, nq : 2 * nq] *= 20  # a key far back that the slow heads still hold at the end
    pos = np.arange(T)
    q = x[:, :nq].reshape(T, heads, dim)
    k = x[:, nq : 2 * nq].reshape(T, heads, dim)
    if rot:
        q, k = Z.rotate_halves(q, pos, rot), Z.rotate_halves(k, pos, rot)
    k = k * dim ** -0.5
    v = x[:, 2 * nq : 2 * nq + nv].reshape(T, heads, vdim)
    out = np.zeros((T, heads, vdim))
    for h in range(heads):
        S = np.zeros((dim, vdim))
        for t in range(T):
            S = decay[h] * S + np.outer(k[t, h], v[t, h])
            out[t, h] = S.T @ q[t, h]
    want = Z.unit_rms(out, eps).reshape(T, nv) * Z.silu(x[:, 2 * nq + nv :])
    cols = {"q": 0, "k": nq, "v": 2 * nq, "g": 2 * nq + nv}
    for cuts in ([230], [30] + [1] * 200, [2, 3, 64, 5, 2, 31, 1, 1, 100, 21]):
        S = torch.full((2, heads, dim, vdim), 3.0, dtype=torch.float32, device=DEV)
        got, at = [], 0
        for c in cuts:
            b = step_batch([c], [at], [1])
            xs = dev(x[at : at + c])
            table = rope_for(o, pos[at : at + c], rot)
            o.rotate_columns_(xs, 0, heads, dim, table, "halves", 1.0)
            o.rotate_columns_(xs, nq, heads, dim, table, "halves", dim ** -0.5)
            y = o.gated_recurrence(xs, cols, heads, dim, vdim, b, {"S": S}, mode="decay", activation=None, decay=dev(decay), chunks=min(decay) > 0)
            got.append(o.group_rmsnorm_gate(y, vdim, None, xs[:, cols["g"] :], eps, torch.float32, "silu"))
            at += c
        close(torch.cat(got), want, torch.float32, f"cuts {cuts[:3]}", 5e-5)


def test_relu_squared():
    o = ops()
    x = np.linspace(-3, 3, 1001)
    close(o.activate(dev(x), "relu_squared", torch.float32), Z.relu_squared(x), torch.float32, tol=1e-6)
    with pytest.raises(NotImplementedError):
        o.gated_linear(dev(np.ones((2, 16))), dev(np.ones((32, 16))), "relu_squared", out_dtype=torch.float32)


@pytest.mark.parametrize("outputs,top,groups,keep", [(1, 1, 1, 1), (3, 3, 1, 1), (8, 2, 4, 2), (16, 4, 4, 3), (24, 4, 6, 3), (70, 8, 7, 2), (300, 5, 1, 1),
                                                     (64, 64, 2, 2), (512, 6, 128, 5), (4, 1, 4, 4), (12, 3, 12, 3)])
def test_routing_by_scores_with_a_correction_and_groups(outputs, top, groups, keep):
    o = ops()
    rng = np.random.default_rng(outputs + top)
    T = 133
    z = (rng.normal(size=(T, outputs)) * 2).astype(np.float32)
    c = (rng.normal(size=outputs) * 0.1).astype(np.float32)
    if outputs > 2:
        z[5] = z[5, 0]  # every score equal: the correction alone decides, and ties go to the lower index
    router = {"experts": outputs, "top": top}
    if groups > 1:
        router["groups"] = {"count": groups, "keep": keep}
    for corr in (dev(c), dev(c, torch.bfloat16), None):
        cc = np.zeros(outputs) if corr is None else corr.float().cpu().numpy().astype(np.float64)
        chosen, weight = Z.route(z.astype(np.float64), {"router": np.eye(outputs), "correction": cc}, router)
        ids, wts = o.moe_route(dev(z), corr, top, "softmax", groups, keep)
        ids, wts = ids.cpu().numpy(), wts.cpu().numpy()
        # a choice may differ where two choice scores lie closer than float32 tells apart
        e = np.exp(z.astype(np.float64) - z.max(-1, keepdims=True))
        s = e / e.sum(-1, keepdims=True)
        for t in range(T):
            if not np.array_equal(ids[t], chosen[t]):
                both = np.sort(np.concatenate([s[t] + cc]))
                assert np.diff(both).min() < 1e-6, f"row {t}: {ids[t]} != {chosen[t]}"
                continue
            assert np.allclose(wts[t], weight[t], rtol=2e-5, atol=1e-7), f"row {t}: weights"
    if outputs > 2 and groups == 1:
        ids, wts = o.moe_route(dev(z), None, top, "softmax", 1, 1)
        assert ids[5].tolist() == list(range(top)) and np.allclose(wts[5].cpu().numpy(), 1.0 / outputs)
    parts = rng.normal(size=(7, T, outputs)).astype(np.float32)
    total = np.zeros((T, outputs), np.float32)
    for part in parts:
        total = total + part
    ids, wts = o.moe_route(o.SplitSum(dev(parts)), dev(c), top, "softmax", groups, keep)
    want_ids, want_wts = o.moe_route(dev(total), dev(c), top, "softmax", groups, keep)
    assert torch.equal(ids, want_ids) and torch.equal(wts, want_wts)
    with pytest.raises(ValueError):
        o.moe_route(dev(z), None, (outputs // groups) * keep + 1, "softmax", groups, keep)


def test_groups_by_hand():
    """Eight outputs in four groups of which two stay: the best output of a group that is left out is not chosen although
    its score is the second largest of all, and the smallest score of a kept group is chosen before it."""
    o = ops()
    s = np.array([[0.30, 0.02, 0.05, 0.25, 0.01, 0.01, 0.28, 0.08]])
    corr = np.array([0.0, 0.0, 0.0, 0.0, 0.0, 0.0, -0.1, -0.3])
    # choice: .30 .02 | .05 .25 | .01 .01 | .18 -.22 ; groups' scores .30 .25 .01 .18 -> groups 0 and 1 stay
    ids, wts = o.moe_route(dev(np.log(s)), dev(corr), 3, "softmax", 4, 2)
    assert ids[0].tolist() == [0, 3, 2] and np.allclose(wts[0].cpu().numpy(), [0.30, 0.25, 0.05], rtol=1e-5)
    chosen, weight = Z.route(np.log(s), {"router": np.eye(8), "correction": corr}, {"experts": 8, "top": 3, "groups": {"count": 4, "keep": 2}})
    assert chosen[0].tolist() == [0, 3, 2] and np.allclose(weight[0], [0.30, 0.25, 0.05])
    ids, _ = o.moe_route(dev(np.log(s)), dev(corr), 4, "softmax", 4, 2)
    assert ids[0].tolist() == [0, 3, 2, 1]  # the fourth comes from the kept groups, however small its score


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,ff,experts,identity,top", [(24, 10, 3, 0, 3), (90, 50, 6, 2, 2), (64, 32, 1, 1, 2), (128, 64, 20, 4, 4), (136, 72, 4, 12, 3),
                                                           (128, 192, 4, 0, 2), (512, 520, 6, 3, 2)])
def test_experts_without_a_gate_and_identity_experts(width, ff, experts, identity, top, dtype):
    """The sorted products against a loop over tokens and choices, for steps of one token to several tiles per expert;
    choices from ``experts`` on give the token's input back, times the weight."""
    o = ops()
    rng = np.random.default_rng(width + experts)
    up, down = rng.normal(size=(experts, ff, width)) / np.sqrt(width), rng.normal(size=(experts, width, ff)) / np.sqrt(ff)
    ur, dr = rounded(up, dtype), rounded(down, dtype)
    for T in (1, 5, 150, 700):
        x = rng.normal(size=(T, width))
        ids = np.stack([rng.permutation(experts + identity)[:top] for _ in range(T)])
        if T == 150:
            ids[:, 0] = ids[0, 0] if ids[0, 0] < experts else 0  # one expert gets every token: several tiles
            for t in range(T):
                for j in range(1, top):
                    while ids[t, j] in ids[t, :j]:
                        ids[t, j] = (ids[t, j] + 1) % (experts + identity)
        wts = rng.random(size=(T, top)) + 0.1
        start = rng.normal(size=(T, width))
        xr = rounded(x, dtype)
        want = start.copy()
        for t in range(T):
            for j in range(top):
                e = ids[t, j]
                if e >= experts:
                    want[t] += np.float32(wts[t, j]) * xr[t]
                    continue
                h = Z.relu_squared(ur[e] @ xr[t])
                if dtype == torch.bfloat16:
                    h = rounded(h, dtype)
                want[t] += np.float32(wts[t, j]) * (dr[e] @ h)
        stream = dev(start)
        o.moe_experts(dev(x, dtype), dev(ids, torch.int32), dev(wts), None, dev(up, dtype), dev(down, dtype), "relu_squared", stream)
        close(stream, want, dtype, f"{T} tokens", tol=3e-5 if dtype == torch.float32 else 6e-3)


# ---------------------------------------------------------------- whole models


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("zigelorn")
    return {name: make_folder(root, name) for name in ZIGELORN}


@pytest.fixture(scope="module")
def plain_logits(folders):
    memo = {}

    def get(name, tokens):
        key = (name, tuple(tokens))
        if key not in memo:
            cfg, w = read_model_folder(folders[name])
            memo[key] = Z.forward(cfg, w, tokens)
        return memo[key]

    return get


def make_runner(folder, dtype, pool_tokens, slots, **kw):
    from miniserve_amd.engine.runner import ModelRunner
    from miniserve_amd.loading import load_model

    return ModelRunner(load_model(folder, dtype, DEV), kv_pool_tokens=pool_tokens, max_running=slots, **kw)


def run_schedule(runner, requests, steps):
    """``steps``: lists of ``(request, count)``; every position's logits are asked for. A request is admitted at its
    first entry and released when its last token has run. Returns request -> ``[T, vocab]``."""
    from miniserve_amd.engine.batch import StepRow

    at = {r: 0 for r in requests}
    live, got = {}, {r: [] for r in requests}
    for step in steps:
        rows, who = [], []
        for r, n in step:
            if r not in live:
                live[r] = runner.acquire()
            rows.append(StepRow(live[r], requests[r][at[r] : at[r] + n], list(range(n))))
            who += [r] * n
            at[r] += n
        logits = runner.step(rows).cpu().numpy()
        for r, row in zip(who, logits):
            got[r].append(row)
        for r, _ in step:
            if at[r] == len(requests[r]):
                runner.release(live.pop(r))
    assert not live and all(at[r] == len(requests[r]) for r in requests)
    return {r: np.stack(v) for r, v in got.items()}


def portions(total, sizes):
    out, i = [], 0
    while total > 0:
        n = min(sizes[i % len(sizes)], total)
        out.append(n)
        total -= n
        i += 1
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(ZIGELORN))
def test_schedules_agree_with_plain(name, dtype, folders, plain_logits):
    """One sequence that passes every window several times: whole, decoded token by token behind a short prefix, and in
    portions of changing sizes down to two tokens and one, through a pool hardly larger than the request."""
    toks = tokens_for(folders[name], 150, 1)
    want = plain_logits(name, toks)
    runner = make_runner(folders[name], dtype, 160, 2)
    seen = {}
    for label, cuts in (("whole", [150]), ("decode", [20] + [1] * 130), ("first token alone", [1, 149]), ("two, then one by one", [2] + [1] * 148),
                        ("portions", portions(150, [2, 3, 17, 64, 5, 2, 31, 1, 1]))):
        got = run_schedule(runner, {"a": toks}, [[("a", n)] for n in cuts])["a"]
        check_logits(got, want, dtype, f"{name} {label}")
        seen[label] = got
        assert runner.cache.idle
    if dtype == "float32":  # cuts change nothing beyond rounding
        for label, got in seen.items():
            assert np.abs(got - seen["whole"]).max() <= 3e-5 * np.abs(want).max(), label


def test_a_router_that_reads_the_whole_stream(tmp_path, folders):
    """The test models' routers read channels that hold the embedding alone. Here the router's weights are random over the
    whole width and the norms behind the sublayers reach every channel; in float32 the choice is still the plain
    implementation's."""
    from safetensors.torch import load_file, save_file

    name = "zgA"
    src = load_file(str(folders[name] / "model.safetensors"))
    gen = torch.Generator().manual_seed(3)
    for k in list(src):
        if k.endswith(".router"):
            src[k] = (torch.randn(src[k].shape, generator=gen) * 0.5).to(torch.bfloat16)
        if k.endswith("norm1b") or k.endswith("norm2b"):
            src[k] = (torch.rand(src[k].shape, generator=gen) * 0.4 - 0.2).to(torch.bfloat16)
    folder = tmp_path / "free"
    folder.mkdir()
    (folder / "config.json").write_text((folders[name] / "config.json").read_text())
    save_file(src, str(folder / "model.safetensors"))
    cfg, w = read_model_folder(folder)
    toks = np.random.default_rng(2).integers(0, cfg["vocab"], size=120).tolist()
    runner = make_runner(folder, "float32", 128, 1)
    got = run_schedule(runner, {"a": toks}, [[("a", n)] for n in portions(120, [33, 1, 2, 50])])["a"]
    check_logits(got, Z.forward(cfg, w, toks), "float32", "a router over the whole stream")


@pytest.mark.parametrize("name", sorted(set(ZIGELORN) - {"zgE"}))  # (zgE's ones leave some options without effect, on purpose)
def test_the_models_show_what_is_left_out(name, folders, plain_logits):
    """What the comparisons are worth: with these weights a window one token off, a missing bias, gate, bonus or
    correction, plain frequencies for slowed ones, a decay that is a little off, the previous token left out of a blend,
    one choice fewer, identity experts that return nothing or a layer that shares another's state moves the logits by far
    more than the tolerance."""
    cfg, w = read_model_folder(folders[name])
    toks = tokens_for(folders[name], 150, 1)
    want = plain_logits(name, toks)
    floor = 50 * 1e-4 * np.abs(want).max()

    def moved(c=cfg, weights=w):
        return np.abs(Z.forward(c, weights, toks) - want).max()

    def without(key, value=0.0):
        out = dict(w)
        out[key] = np.zeros_like(w[key]) + value
        return out

    def other(i, change):
        """The configuration with ``change`` applied to its layer ``i`` (and to the layers that run its weights)."""
        off = copy.deepcopy(cfg)
        for j, layer in enumerate(off["layers"]):
            if j == i or layer.get("weights_of") == i:
                change(layer)
        return off

    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        m, mlp, p = layer["mixer"], layer.get("mlp"), f"l{i}."
        if layer["type"] == "attention":
            if m.get("mask"):
                assert moved(other(i, lambda l: l["mixer"]["mask"].update(size=l["mixer"]["mask"]["size"] - 1))) > floor, (name, i, "window")
            for key in ("mix.q.b", "mix.k.b", "mix.g"):
                assert moved(weights=without(p + key)) > floor, (name, i, key)
            if m.get("rot") and m["rot"].get("scaling") and m["rot"]["scaling"]["factor"] != 1.0:
                assert moved(other(i, lambda l: l["mixer"]["rot"].pop("scaling"))) > floor, (name, i, "slowed frequencies")
        elif layer["type"] == "retention":
            assert moved(other(i, lambda l: l["mixer"].update(decay=[d * 0.98 for d in l["mixer"]["decay"]]))) > floor, (name, i, "decay")
            if m.get("rot"):
                assert moved(other(i, lambda l: l["mixer"].pop("rot"))) > floor, (name, i, "rotation")
        else:
            for key in ("mix.u", "mix.mu.k", "mix.mu.w", "mix.w2"):
                assert moved(weights=without(p + key)) > floor, (name, i, key)
        if mlp and mlp["kind"] == "moe":
            r = mlp["router"]
            outputs = r["experts"] + r.get("identity", 0)
            if r["top"] < outputs:
                assert moved(weights=without(p + "mlp.correction")) > floor, (name, i, "correction")
            if r["top"] > 1:
                assert moved(other(i, lambda l: l["mlp"]["router"].update(top=l["mlp"]["router"]["top"] - 1))) > floor, (name, i, "choices")
            if r.get("groups") and r["groups"]["keep"] < min(r["top"], r["groups"]["count"]):  # (the best k outputs lie in the best k groups)
                assert moved(other(i, lambda l: l["mlp"]["router"].pop("groups"))) > floor, (name, i, "groups")


def random_config(seed):
    """A configuration drawn at random: any order of the mixers, any sizes (odd ones among them), layers that run an
    earlier layer's weights, with and without rotation, window, groups, identity experts and feed-forward."""
    from zigelorn_models import again, attention, dense, model, moe, retention, slowed, wkv

    rng = np.random.default_rng(seed)
    pick = lambda *a: a[int(rng.integers(0, len(a)))]
    width = int(pick(48, 72, 100, 136, 200))
    layers = []
    for i in range(int(rng.integers(2, 7))):
        if layers and rng.random() < 0.25:
            layers.append(again(layers, int(pick(*[j for j, l in enumerate(layers) if l.get("weights_of") is None]))))
            continue
        outputs = int(pick(2, 4, 6, 12, 16))
        count = int(pick(*[c for c in (1, 2, 3, 4) if outputs % c == 0]))
        keep = int(rng.integers(1, count + 1))
        identity = int(pick(0, 0, 1, outputs // 2))
        top = int(rng.integers(1, min(6, outputs // count * keep) + 1))
        mlp = pick(None, dense(int(pick(40, 96, 130))),
                   moe(outputs - identity, top, int(pick(16, 40, 72)), identity=identity, groups=(count, keep) if count > 1 or rng.random() < 0.5 else None))
        kind = pick("attention", "retention", "wkv")
        if kind == "attention":
            kv = int(pick(1, 2, 3))
            dim = int(pick(8, 12, 20, 32, 48, 64, 80))
            dims = int(pick(2, dim // 2 // 2 * 2, dim))
            rot = pick(None, {"base": 200.0, "dims": dims}, slowed(1000.0, dims, float(pick(2.0, 8.0)), int(pick(16, 64)), 8.0, 1.0))
            layers.append(attention(kv * int(pick(1, 2, 4)), kv, dim, float(pick(0.1, 0.3, dim ** -0.5)), rot, pick(None, 1, 5, 16, 33, 70), mlp))
        elif kind == "retention":
            heads, dim = int(pick(1, 3, 4)), int(pick(6, 16, 40, 64, 136))
            dims = int(pick(2, dim // 2 // 2 * 2, dim))
            decay = [float(1.0 - 2.0 ** -rng.uniform(1, 9)) for _ in range(heads)]
            layers.append(retention(heads, dim, int(pick(8, 24, 64, 130)), decay, pick(None, {"base": 100.0, "dims": dims}), mlp))
        else:
            layers.append(wkv(int(pick(1, 2, 5)), int(pick(6, 16, 32, 64, 72)), int(pick(1, 7, 32)), mlp))
    return model(int(pick(50, 131, 300)), width, float(pick(1e-6, 1e-5, 1e-3)), layers)


@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_at_random(seed, tmp_path):
    """Random sizes and orders in float32, where a router's choice needs no help: whole, in portions, decoded, and two
    requests side by side, against the plain implementation."""
    from miniserve_amd.weights.random_init import Init, write_model_folder

    cfg = random_config(seed)
    folder = write_model_folder(tmp_path / "m", cfg, seed, Init(0.15, (0.6, 1.4)))
    cfg, w = read_model_folder(folder)
    rng = np.random.default_rng(seed)
    reqs = {"a": rng.integers(0, cfg["vocab"], size=90).tolist(), "b": rng.integers(0, cfg["vocab"], size=41).tolist()}
    want = {r: Z.forward(cfg, w, t) for r, t in reqs.items()}
    runner = make_runner(folder, "float32", 16 * 10, 2)
    for steps in ([[("a", 90)], [("b", 41)]], [[("a", 37), ("b", 2)], [("a", 1), ("b", 20)], [("a", 2), ("b", 1)]] + [[("a", 1), ("b", 1)]] * 18 +
                  [[("a", 32)]]):
        got = run_schedule(runner, reqs, steps)
        assert runner.cache.idle
        for r in reqs:
            check_logits(got[r], want[r], "float32", f"seed {seed} request {r}: {[l['type'] for l in cfg['layers']]}")
    # bfloat16 runs the same sizes through other kernels. Where no router could choose otherwise for a rounded input the
    # logits are held to the plain implementation's, by the measure of what rounding alone does to these weights at each
    # position (random weights of this spread make single positions several times as touchy as the rest); elsewhere they
    # are at least numbers.
    runner = make_runner(folder, "bfloat16", 16 * 10, 2)
    got = run_schedule(runner, reqs, [[("a", 37), ("b", 2)], [("a", 1), ("b", 20)], [("a", 2), ("b", 1)]] + [[("a", 1), ("b", 1)]] * 18 + [[("a", 32)]])
    routed = any((layer.get("mlp") or {}).get("kind") == "moe" for layer in cfg["layers"])
    for r in reqs:
        assert np.isfinite(got[r]).all()
        if not routed:
            check_logits_against_rounding(got[r], want[r], Z.forward(cfg, w, reqs[r], rounding=Z.to_bfloat16), f"seed {seed} request {r} in bfloat16")


def test_weights_of_a_later_layer_and_through_another(tmp_path):
    """The first layer runs the last layer's weights, the third runs the first's (and so the last's): three states, one
    set of tensors."""
    import copy

    from miniserve_amd.weights.random_init import Init, write_model_folder

    cfg = copy.deepcopy(ZIGELORN["zgC"][0])
    first = cfg["layers"][0]
    cfg["layers"] = [dict(copy.deepcopy(first), weights_of=3), cfg["layers"][1], dict(copy.deepcopy(first), weights_of=0), first]
    folder = write_model_folder(tmp_path / "m", cfg, 3, Init(0.15, (0.6, 1.4)))
    cfg, w = read_model_folder(folder)
    assert not any(k.startswith(("l0.", "l2.")) for k in w)
    toks = np.random.default_rng(0).integers(0, cfg["vocab"], size=70).tolist()
    runner = make_runner(folder, "float32", 128, 1)
    got = run_schedule(runner, {"a": toks}, [[("a", n)] for n in portions(70, [20, 1, 1, 2, 30])])["a"]
    check_logits(got, Z.forward(cfg, w, toks), "float32", "weights of a later layer")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(ZIGELORN))
def test_unequal_requests_in_one_batch_with_pages_and_slots_used_again(name, dtype, folders, plain_logits):
    """Five requests through three slots and a pool that never holds them all: portions of some beside single tokens of
    others, a request of one token, requests admitted into slots and pages that others gave back."""
    lens = {"a": 150, "b": 37, "c": 1, "d": 70, "e": 33}
    reqs = {r: tokens_for(folders[name], n, 10 + i) for i, (r, n) in enumerate(lens.items())}
    steps = [
        [("a", 29)], [("a", 2), ("b", 3)], [("a", 16), ("b", 30), ("c", 1)], [("a", 1), ("b", 1), ("d", 33)],
        [("a", 64), ("b", 1), ("d", 1)], [("b", 1), ("d", 2), ("a", 1)], [("b", 1), ("d", 30), ("a", 7)], [("a", 1), ("d", 1), ("e", 2)],
    ] + [[("a", 1), ("d", 1), ("e", 1)] for _ in range(3)] + [[("a", 26), ("e", 28)]]
    runner = make_runner(folders[name], dtype, 16 * 18, 3)
    got = run_schedule(runner, reqs, steps)
    assert runner.cache.idle
    for r in reqs:
        check_logits(got[r], plain_logits(name, reqs[r]), dtype, f"{name} request {r}")
    with pytest.raises(Exception):
        for _ in range(4):
            runner.acquire()


@pytest.mark.parametrize("name", ["zgB", "zgC"])
def test_long_decoding_through_a_small_pool(name, folders, plain_logits):
    """300 tokens one by one: the windowed groups' pages go round many times, the states run long."""
    toks = tokens_for(folders[name], 300, 7)
    runner = make_runner(folders[name], "float32", 16 * 4, 1)
    got = run_schedule(runner, {"a": toks}, [[("a", 1)] for _ in toks])["a"]
    check_logits(got, plain_logits(name, toks), "float32", "long decoding")
    assert runner.cache.idle


@pytest.mark.parametrize("name", sorted(ZIGELORN))
@pytest.mark.parametrize("chunk,graph", [(0, True), (16, True), (16, False)])
def test_greedy_generation_through_the_engine(name, chunk, graph, folders):
    from miniserve_amd.engine.engine import Engine
    from miniserve_amd.engine.request import SamplingParams
    from miniserve_amd.loading import load_model

    cfg, w = read_model_folder(folders[name])
    prompts = [tokens_for(folders[name], n, 20 + n) for n in (1, 9, 40, 17, 26)]
    want = [Z.greedy(cfg, w, p, 12) for p in prompts]
    eng = Engine(load_model(folders[name], "float32", DEV), kv_pool_tokens=16 * 14, max_running=3, chunked_prefill_size=chunk,
                 decode_graph=graph)
    assert eng.generate(prompts, SamplingParams(max_new_tokens=12)) == want
    assert eng.runner.cache.idle


def test_captured_decode_steps_replay_in_bfloat16(folders, plain_logits):
    """Decode steps of a batch as captured graphs, several replays with other tokens, other experts and states that move."""
    name = "zgD"
    reqs = {r: tokens_for(folders[name], 90, 40 + i) for i, r in enumerate("abc")}
    steps = [[(r, 30) for r in reqs]] + [[(r, 1) for r in reqs] for _ in range(60)]
    runner = make_runner(folders[name], "bfloat16", 16 * 20, 3, decode_graph=True)
    got = run_schedule(runner, reqs, steps)
    assert runner.graph_steps >= 50
    for r in reqs:
        check_logits(got[r], plain_logits(name, reqs[r]), "bfloat16", f"request {r}")


def test_trace_replay(folders, plain_logits, tmp_path):
    from replay_util import Replay

    name = "zgA"
    a, b = tokens_for(folders[name], 70, 31), tokens_for(folders[name], 21, 32)
    with Replay(folders[name], "float32", tmp_path / "out", 128) as run:
        got = [run.step([("a", a[:33], [0, 32])]),
               run.step([("a", a[33:35], [1]), ("b", b, [20])], end=["b"]),
               run.step([("a", a[35:], [34])], end=["a"]),
               run.step([("c", b, [3, 20])], end=["c"])]
        assert run.close() == 0
    wa, wb = plain_logits(name, a), plain_logits(name, b)
    check_logits(np.concatenate(got), np.stack([wa[0], wa[32], wa[34], wb[20], wa[69], wb[3], wb[20]]), "float32", "trace replay")


def test_command_line_random_weights_generate_and_stress(tmp_path):
    """The command line serves the architecture like any other: a folder of random weights from the named preset,
    greedy generation from it against the plain implementation, and a sampled load that returns every page and slot."""
    import json
    import subprocess
    import sys

    from replay_util import ROOT

    folder = tmp_path / "m"
    run = lambda *a: subprocess.run([sys.executable, "-m", "miniserve_amd", *a], capture_output=True, text=True, cwd=str(ROOT), timeout=110)
    res = run("random-weights", "--preset", "zigelorn-tiny", "--seed", "5", "--std", "0.1", "--norm-range", "0.6", "1.4", "--out", str(folder))
    assert res.returncode == 0, res.stderr[-2000:]
    cfg, w = read_model_folder(folder)
    prompt = np.random.default_rng(8).integers(0, cfg["vocab"], size=30).tolist()
    res = run("generate", "--model", str(folder), "--dtype", "float32", "--prompt-ids", ",".join(map(str, prompt)),
              "--max-new-tokens", "8", "--kv-pool-tokens", "256")
    assert res.returncode == 0, res.stderr[-2000:]
    assert json.loads(res.stdout.strip().splitlines()[-1])["outputs"] == [Z.greedy(cfg, w, prompt, 8)]
    res = run("stress", "--model", str(folder), "--num-requests", "12", "--prompt-len", "4", "90", "--max-new-tokens", "1", "20",
              "--kv-pool-tokens", "640", "--max-running", "4", "--chunked-prefill-size", "64", "--temperature", "0.7", "--top-p", "0.9")
    assert res.returncode == 0, res.stdout[-1000:] + res.stderr[-2000:]
    report = json.loads(res.stdout.strip().splitlines()[-1])
    assert report["finished"] == 12 and report["idle"] and report["engine"]["architecture"] == "Zigelorn"
