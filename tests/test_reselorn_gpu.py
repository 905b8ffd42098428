"""Reselorn on the GPU against the plain implementation (``tests/plain/reselorn_plain.py``): every mechanism alone on
inputs made so that a fault shows, then whole models with random weights under every kind of schedule: whole prompts,
token-by-token decoding, portions down to two tokens, batches of unequal requests, pages and slots that are given back
and used again, long decoding, greedy generation through the engine and its scheduler, and the trace replay tool."""

from __future__ import annotations

import copy
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from plain import reselorn_plain as R
from plain.model_folder import read_model_folder
from reselorn_models import RESELORN, make_folder
from tolerances import check_logits

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


def step_batch(lens, starts):
    """What the kernels read of a step: rows of ``lens`` new tokens behind ``starts`` cached ones."""
    pos = np.concatenate([np.arange(s, s + n) for n, s in zip(lens, starts)])
    row = np.concatenate([np.full(n, i) for i, n in enumerate(lens)])
    flat = np.arange(int(sum(lens)))
    single = np.concatenate([np.full(n, n == 1) for n in lens])
    n_dec = int(single.sum())
    mixed = 0 < n_dec < len(flat)
    b = SimpleNamespace(num_rows=len(lens), num_tokens=int(sum(lens)), positions=dev(pos, torch.int32), token_row=dev(row, torch.int32),
                        row_start=dev(np.concatenate(([0], np.cumsum(lens))), torch.int32), starts=dev(starts, torch.int32),
                        state_slots=dev(list(range(len(lens))), torch.int32),
                        num_decode_tokens=n_dec, decode_tokens=dev(flat[single], torch.int32) if mixed else None,
                        prefill_tokens=dev(flat[~single], torch.int32) if mixed else None,
                        max_kv_len=max(s + n for n, s in zip(lens, starts)), row_lens=list(lens), row_starts_host=list(starts), memo={})
    b.is_decode = n_dec == len(flat)
    return b


# ---------------------------------------------------------------- mechanisms alone


def test_rotation_table_with_a_magnitude():
    o = ops()
    pos = np.array([0, 1, 7, 300, 4095])
    f = np.array([1.0, 0.31, 0.004], dtype=np.float32)
    for mag in (1.0, 1.1386):
        got = o.rope_table(dev(pos, torch.int32), dev(f), mag)
        ang = (pos[:, None].astype(np.float32) * f).astype(np.float64)  # the angle itself is a float32 product
        close(got, np.concatenate([np.cos(ang), np.sin(ang)], axis=1) * mag, torch.float32, tol=3e-6)


def plain_prepare(x, pos, hq, hk, d, e, rot, order, qw, kw, eps, v_first, lam):
    """What lies between projection and attention, float64: ``x [T, hq d + hk d + hk e]`` -> queries ``[T, hq, d]``, keys
    ``[T, hk, d]``, values ``[T, hk, e]``. ``rot``: ``(dims, base, scaling, pairing)`` or None."""
    T = x.shape[0]
    q, k = x[:, : hq * d].reshape(T, hq, d), x[:, hq * d : (hq + hk) * d].reshape(T, hk, d)
    v = x[:, (hq + hk) * d :].reshape(T, hk, e)

    def turn(u):
        if rot is None:
            return u
        dims, base, scaling, pairing = rot
        if pairing == "halves":
            return R.rotate_halves(u, pos, {"dims": dims, "base": base, "scaling": scaling})
        f, mag = R.slowed_frequencies(dims, base, scaling)
        ang = pos.astype(np.float64)[:, None] * f
        cos, sin = (np.cos(ang) * mag)[:, None, :], (np.sin(ang) * mag)[:, None, :]
        out = u.copy()
        a, b = u[..., 0:dims:2], u[..., 1:dims:2]
        out[..., 0:dims:2], out[..., 1:dims:2] = a * cos - b * sin, b * cos + a * sin
        return out

    def norm(u, w):
        return R.unit_rms(u, eps) * (1.0 if w is None else w)

    if order == "before":
        q, k = turn(norm(q, qw)), turn(norm(k, kw))
    elif order == "after":
        q, k = norm(turn(q), qw), norm(turn(k), kw)
    else:
        q, k = turn(q), turn(k)
    if v_first is not None:
        v = R.blend_values(v, v_first.reshape(T, hk, e), lam)
    return q, k, v


def rope_for(o, pos, rot):
    if rot is None:
        return None
    dims, base, scaling, _ = rot
    f, mag = R.slowed_frequencies(dims, base, scaling)
    return o.rope_table(dev(pos, torch.int32), dev(f.astype(np.float32)), mag)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hq,hk,d,e,rot,order,weights,blend", [
    (4, 2, 16, 24, (8, 500.0, {"factor": 4.0, "original": 32, "fast": 4.0, "slow": 0.5}, "halves"), "after", False, True),
    (3, 1, 10, 6, (6, 300.0, None, "halves"), "after", False, False),
    (2, 2, 272, 16, (272, 1e4, None, "halves"), "after", True, True),
    (6, 3, 64, 64, (32, 1e3, {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 1.0}, "adjacent"), "before", True, False),
    (2, 1, 70, 9, None, "after", False, True),
    (5, 5, 12, 40, (12, 50.0, {"factor": 2.0, "original": 16, "fast": 2.0, "slow": 0.5}, "halves"), None, False, True),
    (1, 1, 600, 300, (2, 10.0, None, "adjacent"), "before", False, False),
])
def test_rotation_norm_blend_and_store(hq, hk, d, e, rot, order, weights, blend, dtype):
    """The one kernel between projection and attention, every option: the norm before the rotation, behind it (they differ
    where cosines and sines carry a magnitude and only a part of the head is turned) or absent, with weights and without,
    values blended or not. One token's head is tiny against eps, so eps under the root shows."""
    o = ops()
    rng = np.random.default_rng(hq * d + e)
    T, eps, lam = 37, 1e-3, 0.37
    x = rng.normal(size=(T, hq * d + hk * d + hk * e))
    x[3, : d] *= 1e-3
    pos = np.concatenate([np.arange(100, 100 + T - 5), np.arange(5)])
    qw, kw = (rng.normal(size=d) + 1, rng.normal(size=d) + 1) if weights else (None, None)
    wide = rng.normal(size=(T, hk * e + 11))  # the first values are a slice of wider rows
    v_first = wide[:, 5 : 5 + hk * e] if blend else None
    q, k, v = plain_prepare(x, pos, hq, hk, d, e, rot, order, qw, kw, eps, v_first, lam)
    if order == "after" and rot is not None and rot[2] is not None and rot[0] < d:
        other = plain_prepare(x, pos, hq, hk, d, e, rot, "before", qw, kw, eps, v_first, lam)[0]
        assert np.abs(other - q).max() > 0.01  # the place of the norm matters
    slots = rng.permutation(4 * PAGE)[:T]
    kc = torch.zeros((5, hk, PAGE, d), dtype=dtype, device=DEV)
    vc = torch.zeros((5, hk, e, PAGE), dtype=dtype, device=DEV)
    first = dev(wide)[:, 5 : 5 + hk * e] if blend else None
    got = o.head_prepare_store(dev(x), dev(slots, torch.int32), order, None if qw is None else dev(qw), None if kw is None else dev(kw), eps,
                               rope_for(o, pos, rot), rot[3] if rot else "halves", kc, vc, hq, hk, d, e, dtype, first, lam)
    tol = 2e-5 if dtype == torch.float32 else 5e-3
    close(got, q.reshape(T, -1), dtype, "queries", tol)
    at = dev(slots, torch.int64)
    close(kc.permute(0, 2, 1, 3).reshape(-1, hk, d)[at], k, dtype, "keys", tol)
    close(vc.permute(0, 3, 1, 2).reshape(-1, hk, e)[at], v, dtype, "values", tol)
    untouched = np.setdiff1d(np.arange(5 * PAGE), slots)
    assert not kc.permute(0, 2, 1, 3).reshape(-1, hk * d)[dev(untouched, torch.int64)].any()
    # a layer that keeps nothing: queries only, the cache stays as it is
    before = kc.clone()
    again = o.head_prepare_store(dev(x), None, order, None if qw is None else dev(qw), None if kw is None else dev(kw), eps,
                                 rope_for(o, pos, rot), rot[3] if rot else "halves", None, None, hq, hk, d, e, dtype)
    assert torch.equal(again, got) and torch.equal(kc, before)


def plain_attention(q, k, v, scale, size, sinks):
    """``q [T, Hq, D]``, ``k [T, Hk, D]``, ``v [T, Hk, E]`` of one sequence, float64."""
    T, H, _ = q.shape
    per = H // k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for a in range(H):
        s = (q[:, a] @ k[:, a // per].T) * scale
        out[:, a] = R.sink_softmax(s, R.sliding(T, size), float(sinks[a])) @ v[:, a // per]
    return out


CUTS = ([400], [150] + [1] * 250, [2, 3, 64, 5, 2, 31, 1, 1, 190, 1, 100])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hq,hk,d,e,size,dims", [(4, 2, 32, 24, 37, 16), (3, 1, 10, 6, 16, 6), (8, 2, 96, 32, 100, 32), (6, 3, 64, 64, 0, 64),
                                                 (2, 2, 272, 16, 80, 272), (16, 1, 128, 128, 70, 64), (4, 4, 40, 72, 17, 0),
                                                 (4, 2, 32, 24, 1, 16), (2, 1, 64, 64, 2, 32), (4, 2, 128, 128, 16, 64)])
def test_grouped_attention_behind_the_preparation(hq, hk, d, e, size, dims, dtype):
    """Projection rows through rotation, norm, blend and store into pages, then attention with sinks inside a window, in
    cuts of every kind. Queries and keys have unit length here, so a key stands out by its direction: for the last query
    of every head, the key just inside the window and the key just outside it are that query turned to their places (the
    outer one doubled among the values), and a key far back likewise where every key is seen: a window one token off, a
    lost page or a wrong head pairing shows."""
    o = ops()
    rng = np.random.default_rng(hq * d + size)
    T, scale, eps, lam = 400, 8.0 / d, 1e-5, 0.6
    rot = (dims, 1000.0, {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}, "halves") if dims else None
    per = hq // hk
    x = rng.normal(size=(T, hq * d + hk * d + hk * e))
    for g in range(hk):
        a = g * per  # the group's first query head
        inner, outer = (T - size, T - size - 1) if size else (3 + 5 * g, None)
        for at in (inner, outer):
            if at is not None:
                x[at, (hq + g) * d : (hq + g + 1) * d] = x[T - 1, a * d : (a + 1) * d]
        if outer is not None:
            x[outer, (hq + hk) * d + g * e : (hq + hk) * d + (g + 1) * e] *= 4
    if rot is not None:
        # an equal raw vector at another place is turned by another angle; give the keys the place's own turn back
        pos_all = np.arange(T)
        for g in range(hk):
            for at in ((T - size, T - size - 1) if size else (3 + 5 * g,)):
                raw = x[T - 1, g * per * d : (g * per + 1) * d].reshape(1, 1, d)
                there = R.rotate_halves(raw, np.array([T - 1 - at]), {"dims": dims, "base": rot[1], "scaling": rot[2]})[0, 0]
                x[at, (hq + g) * d : (hq + g + 1) * d] = there  # turned by its place it meets the query turned by T - 1
    sinks = rng.normal(size=hq) + 1
    first = rng.normal(size=(T, hk * e))
    q, k, v = plain_prepare(x, np.arange(T), hq, hk, d, e, rot, "after", None, None, eps, first, lam)
    qr, kr, vr = rounded(q, dtype), rounded(k, dtype), rounded(v, dtype)
    want = plain_attention(qr, kr, vr, scale, size, sinks)
    if size:  # the outer key would take most of the weight if it were seen
        seen = plain_attention(qr, kr, vr, scale, size + 1, sinks)
        assert np.abs(seen - want)[T - 1].max() > 0.2 * np.abs(want[T - 1]).max()
        if size > 1:  # (a window of one token sees itself alone: nothing narrower exists)
            lost = plain_attention(qr, kr, vr, scale, size - 1, sinks)
            assert np.abs(lost - want)[T - 1].max() > 0.05 * np.abs(want[T - 1]).max()
    pages = [int(p) for p in rng.permutation(30)[: -(-T // PAGE)]]
    kc = torch.zeros((31, hk, PAGE, d), dtype=dtype, device=DEV)
    vc = torch.zeros((31, hk, e, PAGE), dtype=dtype, device=DEV)
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
            qs = o.head_prepare_store(dev(x[at : at + n]), dev(slots, torch.int32), "after", None, None, eps,
                                      rope_for(o, np.arange(at, at + n), rot), "halves", kc, vc, hq, hk, d, e, dtype, dev(first[at : at + n]), lam)
            got.append(o.paged_attention(qs, kc, vc, table, b, hq, hk, d, scale, size, e, sinks=dev(sinks)))
            at += n
        close(torch.cat(got), want.reshape(T, -1), dtype, f"cuts {cuts[:3]}", tol)
    if size:  # the last tokens again, with every page before the window gone
        first_live = (T - 20 - size + 1) // PAGE
        gone = [-1 if i < first_live else p for i, p in enumerate(pages)]
        b = step_batch([20], [T - 20])
        got = o.paged_attention(dev(q.reshape(T, -1), dtype)[T - 20 :].contiguous(), kc, vc, dev([gone + [0] * (-len(gone) % 4)], torch.int32),
                                b, hq, hk, d, scale, size, e, sinks=dev(sinks))
        close(got, want.reshape(T, -1)[T - 20 :], dtype, "pages before the window given away", tol)


def test_unequal_rows_in_one_attention_step():
    """Rows of one token beside rows of several in one step: each row's result is what it is alone."""
    o = ops()
    rng = np.random.default_rng(5)
    hq, hk, d, e, size = 6, 2, 24, 16, 20
    lens, starts = [1, 7, 1, 30], [50, 0, 3, 41]
    total = [s + n for s, n in zip(starts, lens)]
    seqs = [(R.unit_rms(rng.normal(size=(t, hq, d)), 0), R.unit_rms(rng.normal(size=(t, hk, d)), 0), rng.normal(size=(t, hk, e))) for t in total]
    sinks = rng.normal(size=hq)
    for dtype in (torch.float32, torch.bfloat16):
        kc = torch.zeros((40, hk, PAGE, d), dtype=dtype, device=DEV)
        vc = torch.zeros((40, hk, e, PAGE), dtype=dtype, device=DEV)
        tables, free = [], list(np.random.default_rng(6).permutation(39))
        for (q, k, v), t in zip(seqs, total):
            pages = [int(free.pop()) for _ in range(-(-t // PAGE))]
            for p in range(t):
                kc[pages[p // PAGE], :, p % PAGE] = dev(k[p], dtype)
                vc[pages[p // PAGE], :, :, p % PAGE] = dev(v[p], dtype)
            tables.append(pages + [0] * (8 - len(pages)))
        b = step_batch(lens, starts)
        qs = np.concatenate([q[s:].reshape(n, -1) for (q, _, _), s, n in zip(seqs, starts, lens)])
        got = o.paged_attention(dev(qs, dtype), kc, vc, dev(tables, torch.int32), b, hq, hk, d, 0.9, size, e, sinks=dev(sinks))
        want = np.concatenate([plain_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), 0.9, size, sinks)[s:].reshape(n, -1)
                               for (q, k, v), s, n in zip(seqs, starts, lens)])
        close(got, want, dtype, tol=2e-5 if dtype == torch.float32 else 8e-3)


@pytest.mark.parametrize("experts,top", [(1, 1), (3, 3), (12, 2), (70, 8), (300, 5), (64, 64)])
def test_routing(experts, top):
    o = ops()
    rng = np.random.default_rng(experts)
    T = 133
    z = rng.normal(size=(T, experts)).astype(np.float32)
    b = rng.normal(size=experts).astype(np.float32) * 0.5
    if experts > 2:
        z[5] = z[5, 0]      # every logit equal before the bias
        z[6, :] = 0.25
    for bias in (dev(b), dev(b, torch.bfloat16), None):
        bb = np.zeros(experts) if bias is None else bias.float().cpu().numpy().astype(np.float64)
        zz = (z.astype(np.float64) + bb).astype(np.float32).astype(np.float64)  # the sum as float32 forms it
        chosen, weight = R.route(zz, {"router": np.eye(experts), "router.b": np.zeros(experts)}, top)
        ids, wts = o.moe_route(dev(z), bias, top)
        assert np.array_equal(ids.cpu().numpy(), chosen), "the chosen experts, largest first, ties to the lower index"
        close(wts, weight, torch.float32, tol=3e-6)
    if experts > 2:  # with no bias row 6 is all ties: the first `top` experts in order, equal weights
        ids, wts = o.moe_route(dev(z), None, top)
        assert ids[6].tolist() == list(range(top)) and np.allclose(wts[6].cpu().numpy(), 1.0 / top)
    # logits that arrive as partial sums of the router's product: the kernel adds them in ascending order
    parts = rng.normal(size=(11, T, experts)).astype(np.float32)
    total = np.zeros((T, experts), np.float32)
    for part in parts:
        total = total + part
    ids, wts = o.moe_route(o.SplitSum(dev(parts)), None, top)
    want_ids, want_wts = o.moe_route(dev(total), None, top)
    assert torch.equal(ids, want_ids) and torch.equal(wts, want_wts)
    with pytest.raises(ValueError):
        o.moe_route(dev(z), None, experts + 1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,ff,experts,top", [(24, 10, 3, 3), (90, 50, 7, 2), (64, 32, 1, 1), (128, 64, 20, 4), (136, 72, 40, 1), (96, 264, 5, 5),
                                                  (128, 192, 4, 2), (192, 64, 3, 1), (512, 520, 6, 2)])
def test_experts(width, ff, experts, top, dtype):
    """The sorted products against a loop over tokens and choices, for steps of one token to several tiles per expert, with
    choices that leave experts idle and choices that send every token to one. Widths that are multiples of 64 run the tiles
    staged through LDS (64 and 128 pairs), with output widths that end inside a tile's columns; widths from 512 on split K
    over a block's waves where the step has few tokens."""
    o = ops()
    rng = np.random.default_rng(width + experts)
    gate, up, down = rng.normal(size=(experts, ff, width)), rng.normal(size=(experts, ff, width)), rng.normal(size=(experts, width, ff))
    gr, ur, dr = rounded(gate, dtype), rounded(up, dtype), rounded(down, dtype)
    for T in (1, 5, 150, 700):
        x = rng.normal(size=(T, width)) * 0.3
        ids = np.stack([rng.permutation(experts)[:top] for _ in range(T)])
        if T == 150:
            ids[:, 0] = ids[0, 0]  # one expert gets every token: several tiles
            for t in range(T):
                for j in range(1, top):
                    while ids[t, j] in ids[t, :j]:
                        ids[t, j] = (ids[t, j] + 1) % experts
        wts = rng.random(size=(T, top)) + 0.1
        start = rng.normal(size=(T, width))
        xr = rounded(x, dtype)
        want = start.copy()
        for t in range(T):
            for j in range(top):
                e = ids[t, j]
                h = R.silu(gr[e] @ xr[t]) * (ur[e] @ xr[t])
                if dtype == torch.bfloat16:
                    h = rounded(h, dtype)
                want[t] += np.float32(wts[t, j]) * (dr[e] @ h)
        stream = dev(start)
        o.moe_experts(dev(x, dtype), dev(ids, torch.int32), dev(wts), dev(gate, dtype), dev(up, dtype), dev(down, dtype), "silu", stream)
        close(stream, want, dtype, f"{T} tokens", tol=3e-5 if dtype == torch.float32 else 6e-3)


@pytest.mark.parametrize("width", [7, 1000, 2048, 9000])
def test_output_norm_with_a_rounded_copy_and_a_cleared_stream(width):
    """``residual += y / rms(y) * w`` where ``y`` is a stream, partial sums, or both; the kernel may also hand back the new
    residual in bfloat16 and leave the stream zero. Widths below, at and beyond what a thread keeps in registers."""
    o = ops()
    rng = np.random.default_rng(width)
    rows = 5
    r, y, w = rng.normal(size=(rows, width)), rng.normal(size=(rows, width)) * 4, rng.normal(size=width) + 1
    parts = rng.normal(size=(13, rows, width))
    for stream, pending in ((y, None), (y, parts), (None, parts)):
        total = (0 if stream is None else y) + (0 if pending is None else parts.sum(0))
        want = r + total / np.sqrt((total ** 2).mean(-1, keepdims=True) + 1e-5) * w
        for copy, clear in ((False, False), (True, True), (False, True), (True, False)):
            res = dev(r)
            st = None if stream is None else dev(stream)
            nxt = torch.full((rows, width), 7.0, dtype=torch.bfloat16, device=DEV) if copy else None
            o.normed_add(res, st, dev(w), 1e-5, None if pending is None else o.SplitSum(dev(parts)), nxt, clear)
            close(res, want, torch.float32, tol=3e-5)
            if copy:
                assert torch.equal(nxt, res.to(torch.bfloat16)), "the copy is the new residual, rounded once"
            if st is not None:
                assert (not clear and torch.equal(st, dev(stream))) or (clear and not st.any()), "the stream afterwards"


# ---------------------------------------------------------------- whole models


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("reselorn")
    return {name: make_folder(root, name) for name in RESELORN}


@pytest.fixture(scope="module")
def plain_logits(folders):
    memo = {}

    def get(name, tokens):
        key = (name, tuple(tokens))
        if key not in memo:
            cfg, w = read_model_folder(folders[name])
            memo[key] = R.forward(cfg, w, tokens)
        return memo[key]

    return get


def decisive_tokens(folder):
    """The token ids whose choice of experts is clear in every mixture of the model (the test models route by the token's
    embedding alone): the last chosen logit and the first one left out lie apart."""
    cfg, w = read_model_folder(folder)
    ok = np.ones(cfg["vocab"], dtype=bool)
    for i, layer in enumerate(cfg["layers"]):
        mlp = layer.get("mlp")
        if mlp and mlp["kind"] == "moe" and mlp["router"]["top"] < mlp["router"]["experts"]:
            z = np.sort(w["embed"] @ w[f"l{i}.mlp.router"].T + w[f"l{i}.mlp.router.b"], axis=1)[:, ::-1]
            top = mlp["router"]["top"]
            ok &= (z[:, top - 1] - z[:, top]) > 0.02
    return np.flatnonzero(ok)


def tokens_for(folder, n, seed):
    pool = decisive_tokens(folder)
    assert len(pool) > 20
    return pool[np.random.default_rng(seed).integers(0, len(pool), size=n)].tolist()


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
@pytest.mark.parametrize("name", sorted(RESELORN))
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
            assert np.abs(got - seen["whole"]).max() <= 2e-5 * np.abs(want).max(), label


def test_a_router_that_reads_the_whole_stream(tmp_path, folders):
    """The test models' routers read channels that hold the embedding alone. Here the router's weights are random over the
    whole width; in float32 the choice is still the plain implementation's."""
    from safetensors.torch import load_file, save_file

    name = "rsA"
    src = load_file(str(folders[name] / "model.safetensors"))
    gen = torch.Generator().manual_seed(3)
    for k in list(src):
        if k.endswith(".router"):
            src[k] = (torch.randn(src[k].shape, generator=gen) * 0.5).to(torch.bfloat16)
        if ".ls" in k:
            src[k] = (torch.rand(src[k].shape, generator=gen) + 0.5).to(torch.bfloat16)
    folder = tmp_path / "free"
    folder.mkdir()
    (folder / "config.json").write_text((folders[name] / "config.json").read_text())
    save_file(src, str(folder / "model.safetensors"))
    cfg, w = read_model_folder(folder)
    toks = np.random.default_rng(2).integers(0, cfg["vocab"], size=120).tolist()
    runner = make_runner(folder, "float32", 128, 1)
    got = run_schedule(runner, {"a": toks}, [[("a", n)] for n in portions(120, [33, 1, 2, 50])])["a"]
    check_logits(got, R.forward(cfg, w, toks), "float32", "a router over the whole stream")


@pytest.mark.parametrize("name", sorted(set(RESELORN) - {"rsE"}))  # (rsE's ones leave some options without effect, on purpose)
def test_the_models_show_what_is_left_out(name, folders, plain_logits):
    """What the comparisons are worth: with these weights a window one token off, a sink left out, values that are not
    blended, plain frequencies for slowed ones, a router without its bias, one choice fewer, a missing shared expert or a missing layer scale moves the logits by far more than the
    tolerance."""
    cfg, w = read_model_folder(folders[name])
    toks = tokens_for(folders[name], 150, 1)
    want = plain_logits(name, toks)
    floor = 50 * 1e-4 * np.abs(want).max()

    def moved(c=cfg, weights=w):
        return np.abs(R.forward(c, weights, toks) - want).max()

    def without(key, value=0.0):
        out = dict(w)
        out[key] = np.zeros_like(w[key]) + value
        return out

    blending = False
    for i, layer in enumerate(cfg["layers"]):
        m, mlp = layer["mixer"], layer.get("mlp")
        off = copy.deepcopy(cfg)
        mo = off["layers"][i]["mixer"]
        if m.get("mask"):
            mo["mask"]["size"] -= 1
            assert moved(off) > floor, (name, i, "window")
            mo["mask"]["size"] += 1
        assert moved(weights=without(f"l{i}.mix.sink", -60.0)) > floor, (name, i, "sink")
        if m["v_mix"] and blending:
            assert moved(weights=without(f"l{i}.mix.vmix")) > floor, (name, i, "blend")
        blending = blending or m["v_mix"]
        if m.get("rot") and m["rot"].get("scaling") and m["rot"]["scaling"]["factor"] != 1.0:  # (a factor of one slows nothing)
            sc = mo["rot"].pop("scaling")
            assert moved(off) > floor, (name, i, "slowed frequencies")
            mo["rot"]["scaling"] = sc
        assert moved(weights=without(f"l{i}.ls1", 1.0)) > floor, (name, i, "layer scale")
        if mlp and mlp["kind"] == "moe":
            if mlp["router"]["experts"] > mlp["router"]["top"]:
                assert moved(weights=without(f"l{i}.mlp.router.b")) > floor, (name, i, "router bias")
            if mlp["router"]["top"] > 1:
                off["layers"][i]["mlp"]["router"]["top"] -= 1
                assert moved(off) > floor, (name, i, "choices")
                off["layers"][i]["mlp"]["router"]["top"] += 1
            if mlp.get("shared"):
                del off["layers"][i]["mlp"]["shared"]
                assert moved(off) > floor, (name, i, "shared expert")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(RESELORN))
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


def test_long_decoding_through_a_small_pool(folders, plain_logits):
    """300 tokens one by one: the windowed groups' pages go round many times."""
    name = "rsB"
    toks = tokens_for(folders[name], 300, 7)
    runner = make_runner(folders[name], "float32", 16 * 4, 1)
    got = run_schedule(runner, {"a": toks}, [[("a", 1)] for _ in toks])["a"]
    check_logits(got, plain_logits(name, toks), "float32", "long decoding")
    assert runner.cache.idle


@pytest.mark.parametrize("name", sorted(RESELORN))
@pytest.mark.parametrize("chunk,graph", [(0, True), (16, True), (16, False)])
def test_greedy_generation_through_the_engine(name, chunk, graph, folders):
    from miniserve_amd.engine.engine import Engine
    from miniserve_amd.engine.request import SamplingParams
    from miniserve_amd.loading import load_model

    cfg, w = read_model_folder(folders[name])
    prompts = [tokens_for(folders[name], n, 20 + n) for n in (1, 9, 40, 17, 26)]
    want = [R.greedy(cfg, w, p, 12) for p in prompts]
    eng = Engine(load_model(folders[name], "float32", DEV), kv_pool_tokens=16 * 14, max_running=3, chunked_prefill_size=chunk,
                 decode_graph=graph)
    assert eng.generate(prompts, SamplingParams(max_new_tokens=12)) == want
    assert eng.runner.cache.idle


def test_captured_decode_steps_replay_in_bfloat16(folders, plain_logits):
    """Decode steps of a batch as captured graphs, several replays with other tokens and other experts each time."""
    name = "rsD"
    reqs = {r: tokens_for(folders[name], 90, 40 + i) for i, r in enumerate("abc")}
    steps = [[(r, 30) for r in reqs]] + [[(r, 1) for r in reqs] for _ in range(60)]
    runner = make_runner(folders[name], "bfloat16", 16 * 20, 3, decode_graph=True)
    got = run_schedule(runner, reqs, steps)
    assert runner.graph_steps >= 50
    for r in reqs:
        check_logits(got[r], plain_logits(name, reqs[r]), "bfloat16", f"request {r}")


def test_trace_replay(folders, plain_logits, tmp_path):
    from replay_util import Replay

    name = "rsA"
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
    res = run("random-weights", "--preset", "reselorn-tiny", "--seed", "5", "--std", "0.1", "--norm-range", "0.6", "1.4", "--out", str(folder))
    assert res.returncode == 0, res.stderr[-2000:]
    cfg, w = read_model_folder(folder)
    prompt = np.random.default_rng(8).integers(0, cfg["vocab"], size=30).tolist()
    res = run("generate", "--model", str(folder), "--dtype", "float32", "--prompt-ids", ",".join(map(str, prompt)),
              "--max-new-tokens", "8", "--kv-pool-tokens", "256")
    assert res.returncode == 0, res.stderr[-2000:]
    assert json.loads(res.stdout.strip().splitlines()[-1])["outputs"] == [R.greedy(cfg, w, prompt, 8)]
    res = run("stress", "--model", str(folder), "--num-requests", "12", "--prompt-len", "4", "90", "--max-new-tokens", "1", "20",
              "--kv-pool-tokens", "640", "--max-running", "4", "--chunked-prefill-size", "64", "--temperature", "0.7", "--top-p", "0.9")
    assert res.returncode == 0, res.stdout[-1000:] + res.stderr[-2000:]
    report = json.loads(res.stdout.strip().splitlines()[-1])
    assert report["finished"] == 12 and report["idle"] and report["engine"]["architecture"] == "Reselorn"
