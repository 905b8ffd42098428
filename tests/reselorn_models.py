"""Small Reselorn configurations for the tests. They differ from one another in every size and option: heads and
key/value heads (grouped, one group, none shared), query/key sizes unlike value sizes, sizes that are no multiple of 8,
heads wider than 256, a rotation over the whole head, over a part of it and none, slowed and plain frequencies, windows
shorter and longer than a page and none at all, blended values that start at the first layer or later, layers that
do not blend, dense layers, mixtures with and without a shared expert, one expert, every expert chosen, one chosen,
layers without a feed-forward, and windows of one token, of two and of exactly a page.

``make_folder`` draws random weights and then makes them telling: sinks and blend weights large enough to matter, and a
router whose choice is exact in every number format (it reads only the stream's last channels, which the layer scales
keep out of every sublayer's reach, so they hold the token's embedding, bit for bit): in bfloat16 a router fed by a
rounded stream would now and then choose another expert than the plain implementation, and the comparison would say
nothing about the kernels."""

from __future__ import annotations

from pathlib import Path

import torch
from safetensors.torch import load_file, save_file

from miniserve_amd.weights.random_init import Init, write_model_folder

ROUTER_CHANNELS = 8  # the stream's last channels: no sublayer writes them, the routers read nothing else


def attention(heads, kv_heads, dim, vdim, scale, rot=None, size=None, v_mix=False, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix}
    if rot is not None:
        m["rot"] = rot
    if size is not None:
        m["mask"] = {"size": size}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    out = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def model(vocab, width, eps, layers):
    return {"architecture": "Reselorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


def slowed(base, dims, factor, original, fast, slow):
    return {"base": base, "dims": dims, "scaling": {"factor": factor, "original": original, "fast": fast, "slow": slow}}


RESELORN = {
    # name: (config, seed, init)
    # blending from the first layer on, a layer in between that does not blend, a layer without a feed-forward
    "rsA": (model(101, 64, 1e-5, [
        attention(4, 2, 16, 24, 0.3, slowed(500.0, 8, 4.0, 32, 4.0, 0.5), size=12, v_mix=True, mlp=dense(96)),
        attention(6, 2, 8, 24, 0.4, slowed(500.0, 8, 4.0, 32, 4.0, 0.5), size=33, v_mix=True, mlp=moe(5, 2, 24, 40)),
        attention(2, 2, 24, 8, 0.25, {"base": 100.0, "dims": 24}, size=20, v_mix=False, mlp=moe(4, 1, 16)),
        attention(4, 2, 16, 24, 0.3, slowed(500.0, 8, 4.0, 32, 4.0, 0.5), size=12, v_mix=True, mlp=None),
    ]), 31, Init(0.12, (0.6, 1.4))),
    # sizes that are multiples of nothing; one key/value head for all; every expert chosen; blending starts late
    "rsB": (model(77, 90, 1e-6, [
        attention(3, 1, 10, 6, 0.5, slowed(300.0, 6, 2.5, 20, 3.0, 1.0), size=7, v_mix=False, mlp=moe(3, 3, 50, 34)),
        attention(2, 1, 14, 6, 0.4, {"base": 300.0, "dims": 6}, size=21, v_mix=True, mlp=dense(50)),
        attention(3, 1, 10, 6, 0.5, slowed(300.0, 10, 16.0, 64, 8.0, 2.0), size=17, v_mix=True, mlp=moe(7, 2, 10, 18)),
    ]), 32, Init(0.12, (0.5, 1.5))),
    # heads wider than 256, every earlier token seen, no rotation at all in one layer, one expert
    "rsC": (model(139, 96, 1e-6, [
        attention(2, 2, 272, 16, 0.06, {"base": 10000.0, "dims": 272}, size=None, v_mix=True, mlp=moe(1, 1, 64, 32)),
        attention(4, 2, 64, 16, 0.125, None, size=64, v_mix=True, mlp=dense(80)),
        attention(4, 4, 8, 40, 0.5, slowed(8.0, 2, 3.0, 16, 2.0, 0.25), size=None, v_mix=False, mlp=moe(6, 4, 24)),
    ]), 33, Init(0.1, (0.7, 1.3))),
    # sizes that the matrix-core kernels take; more experts than a tile has rows
    "rsD": (model(160, 128, 1e-5, [
        attention(8, 2, 64, 32, 0.12, slowed(1000.0, 32, 8.0, 64, 16.0, 1.0), size=40, v_mix=True, mlp=moe(20, 4, 64, 64)),
        attention(4, 1, 32, 64, 0.18, slowed(1000.0, 16, 8.0, 64, 16.0, 1.0), size=24, v_mix=False, mlp=dense(192)),
        attention(4, 2, 96, 32, 0.1, {"base": 1000.0, "dims": 32}, size=40, v_mix=True, mlp=moe(9, 3, 32, None)),
        attention(2, 2, 128, 32, 0.09, slowed(1000.0, 64, 2.0, 48, 4.0, 0.5), size=50, v_mix=True, mlp=dense(64)),
    ]), 34, Init(0.1, (0.6, 1.4))),
    # values that are one: a window of a single token and of two, one rotated pair, one chosen expert of two, every one of
    # three, one head, a factor that slows nothing, a window of exactly a page
    "rsE": (model(53, 40, 1e-4, [
        attention(2, 1, 8, 8, 1.0, {"base": 50.0, "dims": 2}, size=1, v_mix=True, mlp=moe(2, 1, 8, 8)),
        attention(2, 2, 8, 8, 0.7, slowed(50.0, 8, 1.0, 8, 1.0, 1.0), size=2, v_mix=False, mlp=moe(3, 3, 8)),
        attention(1, 1, 16, 8, 0.5, None, size=16, v_mix=True, mlp=dense(8)),
    ]), 35, Init(0.15, (0.6, 1.4))),
}


def make_telling(folder: Path, cfg: dict, seed: int) -> None:
    gen = torch.Generator().manual_seed(seed + 1000)
    file = folder / "model.safetensors"
    t = load_file(str(file))
    r = ROUTER_CHANNELS

    def draw(shape, mean, spread):
        return (torch.randn(shape, generator=gen) * spread + mean).to(torch.bfloat16)

    for i, layer in enumerate(cfg["layers"]):
        t[f"l{i}.mix.sink"] = draw(t[f"l{i}.mix.sink"].shape, 0.5, 1.5)
        if f"l{i}.mix.vmix" in t:
            t[f"l{i}.mix.vmix"] = (torch.rand((), generator=gen) * 0.5 + 0.25).to(torch.bfloat16)
        for name in (f"l{i}.ls1", f"l{i}.ls2"):
            if name in t:
                t[name][-r:] = 0
        mlp = layer.get("mlp")
        if mlp and mlp["kind"] == "moe":
            router = torch.zeros_like(t[f"l{i}.mlp.router"])
            router[:, -r:] = draw((router.shape[0], r), 0.0, 2.0)
            t[f"l{i}.mlp.router"] = router
            t[f"l{i}.mlp.router.b"] = draw(t[f"l{i}.mlp.router.b"].shape, 0.0, 0.3)
    t["embed"][:, -r:] = draw((t["embed"].shape[0], r), 0.0, 1.0)
    save_file({k: v.contiguous() for k, v in t.items()}, str(file))


def make_folder(tmp: Path, name: str) -> Path:
    cfg, seed, init = RESELORN[name]
    folder = write_model_folder(Path(tmp) / name, cfg, seed, init)
    make_telling(folder, cfg, seed)
    return folder
