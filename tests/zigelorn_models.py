"""Small Zigelorn configurations for the tests. They differ from one another in every size and option: the order of
the three mixers, layers that run another layer's weights over a state of their own, heads and key/value heads
(grouped, one group, none shared), sizes that are multiples of nothing, sizes that the matrix-core kernels take,
rotations over the whole head, a part of it and none, slowed and plain frequencies, windows shorter and longer than a
page, of exactly a page, of one token and two, and none at all, decays of zero and one, dense layers, mixtures with and
without identity experts and groups, one expert, every output chosen, one chosen, layers without a feed-forward, and a
model that keeps no keys at all.

``make_folder`` draws random weights and then makes them telling: biases, gates, bonuses and decays large enough to
matter, and a router whose choice is exact in every number format. It reads only the stream's last channels, which
the norms behind the sublayers keep out of every sublayer's reach (their ``1 + w`` is zero there), so they hold the
token's embedding, bit for bit; what still varies is the factor ``1 / rms`` of the norm in front of the feed-forward,
and ``decisive_tokens`` keeps the tokens whose choice is the same, by a margin, for every factor in the range the model
shows. In bfloat16 a router fed by a rounded stream would otherwise now and then choose another expert than the plain
implementation, and the comparison would say nothing about the kernels."""

from __future__ import annotations

import copy
from pathlib import Path

import numpy as np
import torch
from safetensors.torch import load_file, save_file

from miniserve_amd.weights.random_init import Init, write_model_folder
from plain import zigelorn_plain as Z
from plain.model_folder import read_model_folder

ROUTER_CHANNELS = 8  # the stream's last channels: no sublayer writes them, the routers read nothing else


def attention(heads, kv_heads, dim, scale, rot=None, size=None, mlp=None, **more):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if rot is not None:
        m["rot"] = rot
    if size is not None:
        m["mask"] = {"size": size}
    return {"type": "attention", "mixer": m, "mlp": mlp, **more}


def retention(heads, dim, vdim, decay, rot=None, mlp=None, **more):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot is not None:
        m["rot"] = rot
    return {"type": "retention", "mixer": m, "mlp": mlp, **more}


def wkv(heads, dim, rank, mlp=None, **more):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim, "rank": rank}, "mlp": mlp, **more}


def again(layers, j):
    """Layer ``j`` of ``layers`` once more: its weights, a cache and state of its own."""
    out = copy.deepcopy(layers[j])
    out["weights_of"] = j
    return out


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, identity=0, groups=None):
    router = {"experts": experts, "top": top}
    if identity:
        router["identity"] = identity
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "router": router, "expert": {"ff": ff}}


def model(vocab, width, eps, layers):
    return {"architecture": "Zigelorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


def slowed(base, dims, factor, original, fast, slow):
    return {"base": base, "dims": dims, "scaling": {"factor": factor, "original": original, "fast": fast, "slow": slow}}


def _zga():
    layers = [
        wkv(4, 16, 8, mlp=dense(96)),
        attention(4, 2, 16, 0.3, slowed(500.0, 8, 4.0, 32, 4.0, 0.5), size=12, mlp=moe(5, 3, 24, identity=3, groups=(4, 2))),
        retention(2, 16, 24, [0.9, 0.99], {"base": 100.0, "dims": 16}, mlp=dense(80)),
    ]
    layers += [again(layers, 1), again(layers, 0), retention(4, 8, 8, [0.5, 0.97, 0.8, 1.0], None, mlp=None)]
    return model(101, 64, 1e-5, layers)


def _zgb():
    # sizes that are multiples of nothing; one key/value head for all; every output chosen; groups of which one is kept
    layers = [
        attention(3, 1, 10, 0.5, slowed(300.0, 6, 2.5, 20, 3.0, 1.0), size=7, mlp=moe(3, 3, 50)),
        wkv(3, 10, 5, mlp=moe(6, 2, 10, identity=2, groups=(2, 1))),
        retention(5, 6, 14, [0.7, 0.9, 0.95, 0.99, 0.999], {"base": 300.0, "dims": 4}, mlp=dense(50)),
        attention(2, 2, 14, 0.4, {"base": 300.0, "dims": 14}, size=21, mlp=None),
    ]
    layers.append(again(layers, 2))
    return model(77, 90, 1e-6, layers)


def _zgc():
    # no keys kept anywhere: recurrences alone
    layers = [wkv(2, 24, 12, mlp=dense(64)), retention(3, 12, 20, [0.8, 0.9, 0.96], {"base": 50.0, "dims": 12}, mlp=moe(4, 2, 16, identity=4))]
    layers.append(again(layers, 0))
    return model(64, 72, 1e-5, layers)


def _zgd():
    # sizes that the matrix-core kernels take; every earlier token seen in one layer; more experts than a tile has rows
    return model(400, 128, 1e-5, [
        attention(8, 2, 64, 0.12, slowed(1000.0, 32, 8.0, 64, 16.0, 1.0), size=40, mlp=moe(20, 4, 64, identity=4, groups=(6, 3))),
        wkv(2, 64, 16, mlp=dense(192)),
        attention(4, 1, 128, 0.09, {"base": 1000.0, "dims": 128}, size=None, mlp=moe(9, 3, 32)),
        retention(2, 128, 64, [0.97, 0.995], {"base": 1000.0, "dims": 64}, mlp=dense(64)),
        attention(4, 4, 32, 0.18, slowed(1000.0, 16, 2.0, 48, 4.0, 0.5), size=50, mlp=moe(4, 4, 64, identity=12, groups=(4, 2))),
    ])


def _zge():
    # values that are one: windows of a single token, of two and of exactly a page, one rotated pair, one head, one expert
    # beside one identity expert, a factor that slows nothing, one group, decays of zero and of one
    return model(53, 40, 1e-4, [
        attention(2, 1, 8, 1.0, {"base": 50.0, "dims": 2}, size=1, mlp=moe(1, 1, 8, identity=1)),
        wkv(1, 8, 1, mlp=moe(2, 2, 8, groups=(1, 1))),
        attention(2, 2, 8, 0.7, slowed(50.0, 8, 1.0, 8, 1.0, 1.0), size=2, mlp=moe(3, 1, 8, identity=1, groups=(4, 4))),
        retention(1, 8, 8, [1.0], {"base": 20.0, "dims": 2}, mlp=dense(8)),
        attention(1, 1, 16, 0.5, None, size=16, mlp=dense(8)),
        retention(2, 4, 8, [0.0, 0.5], None, mlp=None),
    ])


ZIGELORN = {
    # name: (config, seed, init)
    "zgA": (_zga(), 41, Init(0.12, (0.6, 1.4))),
    "zgB": (_zgb(), 42, Init(0.12, (0.5, 1.5))),
    "zgC": (_zgc(), 43, Init(0.12, (0.6, 1.4))),
    "zgD": (_zgd(), 44, Init(0.1, (0.6, 1.4))),
    "zgE": (_zge(), 45, Init(0.15, (0.6, 1.4))),
}


def make_telling(folder: Path, cfg: dict, seed: int) -> None:
    gen = torch.Generator().manual_seed(seed + 1000)
    file = folder / "model.safetensors"
    t = load_file(str(file))
    r = ROUTER_CHANNELS

    def draw(shape, mean, spread):
        return (torch.randn(shape, generator=gen) * spread + mean).to(torch.bfloat16)

    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        p = f"l{i}."
        for name in ("norm1b", "norm2b"):
            if p + name in t:
                t[p + name][-r:] = -1.0  # 1 + w = 0: the sublayers add nothing to the router's channels
        if layer["type"] == "attention":
            for name in ("mix.q.b", "mix.k.b"):
                t[p + name] = draw(t[p + name].shape, 0.0, 0.5)
            t[p + "mix.g"] = draw(t[p + "mix.g"].shape, 0.0, 0.4)
        elif layer["type"] == "wkv":
            t[p + "mix.u"] = draw(t[p + "mix.u"].shape, 0.5, 0.5)
            t[p + "mix.w0"] = draw(t[p + "mix.w0"].shape, -2.0, 1.5)  # decays from about 0.4 to nearly one
            t[p + "mix.w2"] = draw(t[p + "mix.w2"].shape, 0.0, 0.5)
            for s in "rkvgw":
                t[p + f"mix.mu.{s}"] = torch.rand(t[p + f"mix.mu.{s}"].shape, generator=gen).to(torch.bfloat16)
        mlp = layer.get("mlp")
        if mlp and mlp["kind"] == "moe":
            router = torch.zeros_like(t[p + "mlp.router"])
            # small logits: the scores stay near 1 / outputs, where a rounded input moves them by a hundredth of the margin
            # that ``decisive_tokens`` asks for; the correction is of the size of the scores' spread
            router[:, -r:] = draw((router.shape[0], r), 0.0, 0.3)
            t[p + "mlp.router"] = router
            t[p + "mlp.correction"] = draw(t[p + "mlp.correction"].shape, 0.0, 0.15 / router.shape[0])
    t["embed"][:, -r:] = draw((t["embed"].shape[0], r), 0.0, 1.0)
    save_file({k: v.contiguous() for k, v in t.items()}, str(file))


def make_folder(tmp: Path, name: str) -> Path:
    cfg, seed, init = ZIGELORN[name]
    folder = write_model_folder(Path(tmp) / name, cfg, seed, init)
    make_telling(folder, cfg, seed)
    return folder


def choice_margin(z, correction, router):
    """Per row of the router logits ``z [N, outputs]``: the chosen outputs (a sorted tuple) and how far the choice is from
    being another, the least of: last kept group against first one left out, last chosen score against the first one
    left out among the kept groups."""
    e = np.exp(z - z.max(axis=-1, keepdims=True))
    c = e / e.sum(axis=-1, keepdims=True) + correction
    margin = np.full(len(z), np.inf)
    groups = router.get("groups")
    if groups and groups["keep"] < groups["count"]:
        n = c.shape[-1] // groups["count"]
        best = c.reshape(len(z), groups["count"], n).max(axis=-1)
        order = np.sort(best, axis=-1)[:, ::-1]
        margin = order[:, groups["keep"] - 1] - order[:, groups["keep"]]
        kept = np.argsort(-best, axis=-1, kind="stable")[:, : groups["keep"]]
        allowed = np.zeros(best.shape, dtype=bool)
        np.put_along_axis(allowed, kept, True, axis=-1)
        c = np.where(np.repeat(allowed, n, axis=-1), c, -np.inf)
    top = router["top"]
    order = np.sort(c, axis=-1)[:, ::-1]
    if top < c.shape[-1] and np.isfinite(order[:, top]).any():
        margin = np.minimum(margin, np.where(np.isfinite(order[:, top]), order[:, top - 1] - order[:, top], np.inf))
    chosen = [tuple(sorted(row)) for row in np.argsort(-c, axis=-1, kind="stable")[:, :top]]
    return chosen, margin


def decisive_tokens(folder, margin=0.03, pilot=160, slack=1.4):
    """The token ids whose choice of experts is the same in every mixture of the model whatever the stream around them
    looks like: the routers read ``embed[token] (1 + norm2) / rms(stream)`` on the router's channels, so the choice is
    looked at for every factor ``1 / rms`` between the extremes a pilot run shows, stretched by ``slack``. ``margin`` is
    in units of ``1 / outputs``, the size of a score."""
    cfg, w = read_model_folder(folder)
    r = ROUTER_CHANNELS
    seen = {}
    toks = np.random.default_rng(99).integers(0, cfg["vocab"], size=pilot)
    Z.forward(cfg, w, toks, watch=lambda i, x: seen.setdefault(i, []).append(1.0 / np.sqrt((x * x).mean(-1) + cfg["norm"]["eps"])))
    ok = np.ones(cfg["vocab"], dtype=bool)
    for i, layer in enumerate(cfg["layers"]):
        mlp = layer.get("mlp")
        if not (mlp and mlp["kind"] == "moe"):
            continue
        p = f"l{layer.get('weights_of', i)}."
        factors = np.concatenate(seen[i])
        lo, hi = factors.min() / slack, factors.max() * slack
        base = (w["embed"][:, -r:] * (1.0 + w[p + "norm2"][-r:])) @ w[p + "mlp.router"][:, -r:].T
        first = None
        for f in np.geomspace(lo, hi, 25):
            chosen, m = choice_margin(base * f, w[p + "mlp.correction"], mlp["router"])
            ok &= m > margin / base.shape[1]
            if first is None:
                first = chosen
            ok &= np.array([a == b for a, b in zip(chosen, first)])
    return np.flatnonzero(ok)


def tokens_for(folder, n, seed):
    pool = decisive_tokens(folder)
    assert len(pool) >= 12, f"only {len(pool)} tokens choose their experts clearly"
    return pool[np.random.default_rng(seed).integers(0, len(pool), size=n)].tolist()
