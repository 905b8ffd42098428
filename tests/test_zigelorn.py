"""Zigelorn on the CPU: its configuration and lowering (layers that run another layer's weights over a state of their
own, what the cache manager makes of windows and states, a tensor size that no key states), and the plain
implementation held against forms that do not share its loops."""

from __future__ import annotations

import copy
import math

import numpy as np
import pytest

from miniserve_amd.cache import CacheLayout
from miniserve_amd.config import config_from_dict
from miniserve_amd.config.presets import preset
from miniserve_amd.parts.base import TensorSpec
from miniserve_amd.parts.model import expected_tensors
from miniserve_amd.parts.registry import part_class
from plain import zigelorn_plain as Z
from plain.model_folder import read_model_folder
from zigelorn_models import ROUTER_CHANNELS, ZIGELORN, choice_margin, decisive_tokens, make_folder, tokens_for


# ---------------------------------------------------------------- configuration


@pytest.mark.parametrize("name", sorted(ZIGELORN))
def test_config_reads_back_and_names_its_tensors(name):
    cfg = ZIGELORN[name][0]
    c = config_from_dict(cfg)
    assert config_from_dict(c.to_dict()).to_dict() == c.to_dict()
    names = expected_tensors(c.to_spec())
    w = cfg["width"]
    assert names["embed"].shape == (cfg["vocab"], w) and names["final.norm"].shape == (w,) and "head" not in names
    for i, layer in enumerate(cfg["layers"]):
        m, mlp, p = layer["mixer"], layer["mlp"], f"l{i}."
        if layer.get("weights_of") is not None:
            assert not any(k.startswith(p) for k in names), "a layer that runs another's weights has no tensors"
            continue
        n = m["heads"] * m["dim"]
        assert names[p + "norm1"].shape == names[p + "norm1b"].shape == (w,)
        assert names[p + "norm2"].optional == names[p + "norm2b"].optional == (not mlp)
        if layer["type"] == "attention":
            g = m["kv_heads"] * m["dim"]
            assert names[p + "mix.q"].shape == (n, w) and names[p + "mix.k"].shape == (g, w) and p + "mix.v" not in names
            assert names[p + "mix.q.b"].shape == names[p + "mix.q.norm"].shape == (n,)
            assert names[p + "mix.k.b"].shape == names[p + "mix.k.norm"].shape == (g,)
            assert names[p + "mix.g"].shape == (m["heads"], w) and names[p + "mix.o"].shape == (w, n)
        elif layer["type"] == "retention":
            e = m["heads"] * m["vdim"]
            assert names[p + "mix.q"].shape == names[p + "mix.k"].shape == (n, w)
            assert names[p + "mix.v"].shape == names[p + "mix.g"].shape == (e, w) and names[p + "mix.o"].shape == (w, e)
            assert p + "mix.norm" not in names
        else:
            for s in "rkvg":
                assert names[p + f"mix.{s}"].shape == (n, w) and names[p + f"mix.mu.{s}"].shape == (w,)
            assert names[p + "mix.w1"].shape == (m["rank"], w) and names[p + "mix.w2"].shape == (n, m["rank"])
            assert names[p + "mix.w0"].shape == names[p + "mix.norm"].shape == (n,) and names[p + "mix.u"].shape == (m["heads"], m["dim"])
        if not mlp:
            assert not any(k.startswith(p + "mlp.") for k in names)
        elif mlp["kind"] == "dense":
            assert names[p + "mlp.up"].shape == (mlp["ff"], w) and names[p + "mlp.down"].shape == (w, mlp["ff"]) and p + "mlp.gate" not in names
        else:
            r = mlp["router"]
            e, outputs, f = r["experts"], r["experts"] + r.get("identity", 0), mlp["expert"]["ff"]
            assert names[p + "mlp.router"].shape == (outputs, w) and names[p + "mlp.correction"].shape == (outputs,)
            assert names[p + f"mlp.e{e - 1}.up"].shape == (f, w) and names[p + "mlp.e0.down"].shape == (w, f)
            assert p + f"mlp.e{e}.up" not in names and p + "mlp.e0.gate" not in names


def test_a_layer_that_runs_anothers_weights_has_a_state_of_its_own():
    cfg = ZIGELORN["zgA"][0]
    spec = config_from_dict(cfg).to_spec()
    assert len(spec.layers) == 4 and [(e.layer, e.cache, e.writes_cache) for e in spec.run_order] == [
        (0, 0, True), (1, 1, True), (2, 2, True), (1, 3, True), (0, 4, True), (3, 5, True)]
    assert [layer.prefix for layer in spec.layers] == ["l0.", "l1.", "l2.", "l5."]


def test_weights_of_a_later_layer_and_through_another():
    """The layer that has the tensors may come later, and may be named through a layer that runs its weights too."""
    cfg = copy.deepcopy(ZIGELORN["zgC"][0])  # wkv, retention, wkv (weights of 0)
    first = cfg["layers"][0]
    cfg["layers"] = [dict(copy.deepcopy(first), weights_of=3), cfg["layers"][1], dict(copy.deepcopy(first), weights_of=0), first]
    spec = config_from_dict(cfg).to_spec()
    assert [layer.prefix for layer in spec.layers] == ["l1.", "l3."]
    assert [(e.layer, e.cache) for e in spec.run_order] == [(1, 0), (0, 1), (1, 2), (1, 3)]
    names = expected_tensors(spec)
    assert "l3.mix.r" in names and not any(k.startswith(("l0.", "l2.")) for k in names)


def test_cache_groups_and_states():
    """Windowed attention layers of one shape share a group; every recurrent layer keeps a state and no pages; a model
    of recurrences alone has no group at all."""
    from miniserve_amd.parts.model import CacheSlotNeed

    def needs(name):
        spec = config_from_dict(ZIGELORN[name][0]).to_spec()
        out = []
        for e in spec.run_order:
            layer = spec.layers[e.layer]
            mixer = part_class("mixer", layer.mixer)(layer.mixer, None)
            out.append(CacheSlotNeed(e.cache, mixer.kv_need(), mixer.state_need()))
        return out

    a = needs("zgA")
    assert [n.kv is not None for n in a] == [False, True, False, True, False, False]
    assert a[1].kv.window == 12 and [p.width for p in a[1].kv.planes] == [16, 16] and a[1].kv == a[3].kv
    assert {t.name: t.shape for t in a[0].state.tensors} == {"S": (4, 16, 16), "shift": (64,)}
    assert {t.name: t.shape for t in a[2].state.tensors} == {"S": (2, 16, 24)} and a[1].state is None
    layout = CacheLayout.from_needs(a)
    assert len(layout.groups) == 1 and layout.groups[0].slots == (1, 3) and layout.groups[0].window == 12
    assert len(CacheLayout.from_needs(needs("zgC")).groups) == 0
    d = CacheLayout.from_needs(needs("zgD"))
    assert sorted(g.window for g in d.groups) == [0, 40, 50]


def test_config_refusals():
    base = ZIGELORN["zgA"][0]

    def broken(change):
        cfg = copy.deepcopy(base)
        change(cfg)
        return cfg

    for change, error in [
        (lambda c: c["layers"][1].update(type="conv"), NotImplementedError),
        (lambda c: c["layers"][1]["mixer"].update(vdim=8), ValueError),            # the values are the keys
        (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), ValueError),
        (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=18), ValueError),
        (lambda c: c["layers"][2]["mixer"].update(decay=[0.9]), ValueError),       # one decay per head
        (lambda c: c["layers"][2]["mixer"].update(decay=[0.9, 1.5]), ValueError),
        (lambda c: c["layers"][3].update(weights_of=9), ValueError),               # no such layer
        (lambda c: c["layers"][3].update(weights_of=3), ValueError),               # itself
        (lambda c: c["layers"][1].update(weights_of=3), ValueError),               # a ring: nobody has the tensors
        (lambda c: c["layers"][3].update(weights_of=0), ValueError),               # a layer of another kind
        (lambda c: c["layers"][1]["mlp"]["router"].update(top=5), ValueError),     # more than the kept groups hold
        (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=3), ValueError),
        (lambda c: c["layers"][1]["mlp"].update(kind="gated"), NotImplementedError),
        (lambda c: c.pop("norm"), KeyError),
    ]:
        with pytest.raises(error):
            config_from_dict(broken(change))


def test_the_preset_and_the_measured_shapes_are_valid_configurations():
    from miniserve_amd.measurement.designs import SHAPES, zigelorn_config

    for cfg in [preset("zigelorn-tiny")] + [zigelorn_config(s) for s in SHAPES.values()]:
        spec = config_from_dict(cfg).to_spec()
        assert spec.architecture == "Zigelorn" and len(spec.run_order) == len(cfg["layers"])
        assert {layer["type"] for layer in cfg["layers"]} == {"attention", "retention", "wkv"}


def test_a_size_that_no_key_states_is_read_off_the_tensors(tmp_path):
    """How wide the decay's first step is only the tensors say: a configuration without ``rank`` declares the dimension
    free, and a checkpoint of any rank fits it."""
    cfg = copy.deepcopy(ZIGELORN["zgC"][0])
    for layer in cfg["layers"]:
        layer["mixer"].pop("rank", None)
    names = expected_tensors(config_from_dict(cfg).to_spec())
    w1, w2 = names["l0.mix.w1"], names["l0.mix.w2"]
    assert w1.shape == (None, 72) and w2.shape == (48, None) and w1.free == w2.free and w1.free >= 1
    assert w1.fits((12, 72)) and w1.fits((3, 72)) and not w1.fits((12, 71)) and not w1.fits((12,))
    assert w1.drawn_shape() == (w1.free, 72)
    with pytest.raises(ValueError):
        TensorSpec((None, 4))


# ---------------------------------------------------------------- the plain implementation against other forms


def test_rotation_turns_halves_and_keeps_the_rest():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(5, 2, 10))
    pos = np.array([0, 1, 2, 50, 7])
    rot = {"dims": 6, "base": 100.0, "scaling": {"factor": 4.0, "original": 16, "fast": 2.0, "slow": 0.5}}
    y = Z.rotate_halves(x, pos, rot)
    f, mag = Z.frequencies(6, 100.0, rot["scaling"])
    assert mag == pytest.approx(0.1 * math.log(4.0) + 1.0)
    assert np.array_equal(y[..., 6:], x[..., 6:]) and np.allclose(y[0], x[0] * np.r_[[mag] * 6, [1.0] * 4])
    for j in range(3):
        z = (x[..., j] + 1j * x[..., j + 3]) * np.exp(1j * pos[:, None] * f[j]) * mag
        assert np.allclose(y[..., j], z.real) and np.allclose(y[..., j + 3], z.imag)
    plain, one = Z.frequencies(6, 100.0, None)
    assert one == 1.0 and np.allclose(plain, 100.0 ** (-np.arange(3) / 3.0))
    assert np.all(f <= plain) and np.all(f >= plain / 4.0)


def test_retention_as_a_sum_over_earlier_tokens():
    """``o_t = sum_(j <= t) decay^(t - j) (q_t . k_j) v_j``: the recurrence written out."""
    rng = np.random.default_rng(1)
    T, W = 30, 24
    m = {"heads": 2, "dim": 6, "vdim": 4, "decay": [0.8, 0.97], "rot": {"base": 30.0, "dims": 4}}
    w = {"q": rng.normal(size=(12, W)), "k": rng.normal(size=(12, W)), "v": rng.normal(size=(8, W)), "g": rng.normal(size=(8, W)),
         "o": rng.normal(size=(W, 8))}
    h = rng.normal(size=(T, W))
    pos = np.arange(T)
    q = Z.rotate_halves((h @ w["q"].T).reshape(T, 2, 6), pos, m["rot"])
    k = Z.rotate_halves((h @ w["k"].T).reshape(T, 2, 6), pos, m["rot"]) / math.sqrt(6)
    v = (h @ w["v"].T).reshape(T, 2, 4)
    out = np.zeros((T, 2, 4))
    for a in range(2):
        d = pos[:, None] - pos[None, :]
        weights = np.where(d >= 0, m["decay"][a] ** np.maximum(d, 0), 0.0) * (q[:, a] @ k[:, a].T)
        out[:, a] = weights @ v[:, a]
    want = (Z.unit_rms(out, 1e-5).reshape(T, 8) * Z.silu(h @ w["g"].T)) @ w["o"].T
    assert np.allclose(Z.retention(h, w, m, 1e-5, pos), want)


def test_wkv_as_a_sum_over_earlier_tokens():
    """``o_t = sum_(j < t) (r_t * prod_(j < i < t) w_i . k_j) v_j + (r_t * u . k_t) v_t``."""
    rng = np.random.default_rng(2)
    T, W, H, D, R = 17, 20, 2, 5, 3
    m = {"heads": H, "dim": D}
    w = {s: rng.normal(size=(H * D, W)) * 0.3 for s in "rkvg"}
    w.update({f"mu.{s}": rng.random(size=W) for s in "rkvgw"})
    w.update({"w1": rng.normal(size=(R, W)), "w2": rng.normal(size=(H * D, R)), "w0": rng.normal(size=H * D) - 1, "u": rng.normal(size=(H, D)),
              "norm": rng.normal(size=H * D) + 1, "o": rng.normal(size=(W, H * D))})
    h = rng.normal(size=(T, W))
    prev = np.vstack([np.zeros((1, W)), h[:-1]])
    mix = {s: h + (prev - h) * w[f"mu.{s}"] for s in "rkvgw"}
    r, k, v = ((mix[s] @ w[s].T).reshape(T, H, D) for s in "rkv")
    decay = np.exp(-np.exp(np.tanh(mix["w"] @ w["w1"].T) @ w["w2"].T + w["w0"])).reshape(T, H, D)
    out = np.zeros((T, H, D))
    for t in range(T):
        for a in range(H):
            acc = (r[t, a] * w["u"][a] * k[t, a]).sum() * v[t, a]
            for j in range(t):
                between = np.prod(decay[j + 1 : t, a], axis=0) if t - j > 1 else np.ones(D)
                acc = acc + (r[t, a] * between * k[j, a]).sum() * v[j, a]
            out[t, a] = acc
    want = (Z.unit_rms(out, 1e-5).reshape(T, H * D) * w["norm"] * Z.silu(mix["g"] @ w["g"].T)) @ w["o"].T
    assert np.allclose(Z.wkv(h, w, m, 1e-5), want)
    # the first token has nothing before it: its blends are (1 - mu) h
    assert np.allclose(Z.shifted(h)[0], 0) and np.allclose(Z.shifted(h)[1:], h[:-1])


def test_attention_of_one_token_returns_its_gated_key_as_projected():
    """A window of one token: the softmax has one term, so the output is the token's own value, which is its key with the
    bias and without norm or rotation, times the gate."""
    rng = np.random.default_rng(3)
    T, W = 6, 12
    m = {"heads": 4, "kv_heads": 2, "dim": 4, "scale": 0.5, "rot": {"base": 10.0, "dims": 4}, "mask": {"size": 1}}
    w = {"q": rng.normal(size=(16, W)), "k": rng.normal(size=(8, W)), "q.b": rng.normal(size=16), "k.b": rng.normal(size=8),
         "q.norm": rng.normal(size=16), "k.norm": rng.normal(size=8), "g": rng.normal(size=(4, W)), "o": np.eye(16)}
    h = rng.normal(size=(T, W))
    key = (h @ w["k"].T + w["k.b"]).reshape(T, 2, 4)
    want = np.repeat(key, 2, axis=1) * Z.sigmoid(h @ w["g"].T)[:, :, None]
    assert np.allclose(Z.attention(h, w, m, 1e-6, np.arange(T)), want.reshape(T, 16))


def test_routing_by_hand():
    s = np.array([[0.30, 0.02, 0.05, 0.25, 0.01, 0.01, 0.28, 0.08]])
    corr = np.array([0.0, 0.0, 0.0, 0.0, 0.0, 0.0, -0.1, -0.3])
    w = {"router": np.eye(8), "correction": corr}
    chosen, weight = Z.route(np.log(s), w, {"experts": 8, "top": 3, "groups": {"count": 4, "keep": 2}})
    assert chosen[0].tolist() == [0, 3, 2] and np.allclose(weight[0], [0.30, 0.25, 0.05])  # group 3's 0.18 is left out
    chosen, weight = Z.route(np.log(s), w, {"experts": 8, "top": 3})
    assert chosen[0].tolist() == [0, 3, 6] and np.allclose(weight[0], [0.30, 0.25, 0.28])  # the weight is the score, not the choice score
    chosen, _ = Z.route(np.log(s), {"router": np.eye(8), "correction": np.zeros(8)}, {"experts": 8, "top": 3})
    assert chosen[0].tolist() == [0, 6, 3]
    tokens, margin = choice_margin(np.log(s), corr, {"experts": 8, "top": 3, "groups": {"count": 4, "keep": 2}})
    assert tokens[0] == (0, 2, 3) and margin[0] == pytest.approx(0.03)  # 0.05 against 0.02; the groups lie 0.07 apart


def test_identity_experts_return_the_input():
    """A mixture whose router can only choose its identity outputs gives every token back, times the scores."""
    rng = np.random.default_rng(4)
    h = rng.normal(size=(7, 10))
    w = {"router": rng.normal(size=(5, 10)), "correction": np.array([-9.0, -9.0, -9.0, 0.0, 0.0]),
         **{f"e{j}.{k}": rng.normal(size=s) for j in range(3) for k, s in (("up", (6, 10)), ("down", (10, 6)))}}
    mlp = {"router": {"experts": 3, "identity": 2, "top": 2}}
    z = h @ w["router"].T
    s = np.exp(z) / np.exp(z).sum(-1, keepdims=True)
    assert np.allclose(Z.mixture_ff(h, w, mlp), h * (s[:, 3] + s[:, 4])[:, None])


def test_a_one_layer_model_in_closed_form(tmp_path):
    """One retention layer without a feed-forward, one token: the state is ``k v^T``, so the head's output is ``(q . k) v``."""
    cfg = {"architecture": "Zigelorn", "vocab": 11, "width": 8, "norm": {"eps": 1e-6},
           "layers": [{"type": "retention", "mixer": {"heads": 1, "dim": 4, "vdim": 8, "decay": [0.5]}, "mlp": None}]}
    rng = np.random.default_rng(5)
    w = {"embed": rng.normal(size=(11, 8)), "final.norm": rng.normal(size=8) * 0.1, "l0.norm1": rng.normal(size=8) * 0.1,
         "l0.norm1b": rng.normal(size=8) * 0.1, "l0.mix.q": rng.normal(size=(4, 8)), "l0.mix.k": rng.normal(size=(4, 8)),
         "l0.mix.v": rng.normal(size=(8, 8)), "l0.mix.g": rng.normal(size=(8, 8)), "l0.mix.o": rng.normal(size=(8, 8))}
    x = w["embed"][3]
    norm = lambda y, g: y / np.sqrt((y * y).mean() + 1e-6) * (1 + g)
    h = norm(x, w["l0.norm1"])
    q, k, v = w["l0.mix.q"] @ h, w["l0.mix.k"] @ h / 2.0, w["l0.mix.v"] @ h
    o = (q @ k) * v
    y = w["l0.mix.o"] @ (o / np.sqrt((o * o).mean() + 1e-6) * Z.silu(w["l0.mix.g"] @ h))
    x = x + norm(y, w["l0.norm1b"])
    assert np.allclose(Z.forward(cfg, w, [3])[0], w["embed"] @ norm(x, w["final.norm"]))


def test_the_test_models_route_by_the_tokens_embedding_alone(tmp_path):
    """What ``make_folder`` promises: no sublayer writes the stream's last channels, so a router that reads only those
    sees the embedding times the norm's factor, and the chosen experts are those ``decisive_tokens`` foresaw."""
    name = "zgA"
    folder = make_folder(tmp_path, name)
    cfg, w = read_model_folder(folder)
    toks = tokens_for(folder, 60, 3)
    assert set(toks) <= set(decisive_tokens(folder).tolist())
    _, layers = Z.forward(cfg, w, toks, return_layers=True)
    r = ROUTER_CHANNELS
    for after in layers:
        assert np.array_equal(after[:, -r:], w["embed"][toks][:, -r:])
    seen = {}
    Z.forward(cfg, w, toks, watch=lambda i, x: seen.setdefault(i, x))
    for i, x in seen.items():
        layer = cfg["layers"][i]
        if layer["mlp"]["kind"] != "moe":
            continue
        p = f"l{layer.get('weights_of', i)}."
        chosen, _ = Z.route(Z.one_plus_norm(x, w[p + "norm2"], cfg["norm"]["eps"]), {k[len(p) + 4:]: v for k, v in w.items() if k.startswith(p + "mlp.")},
                            layer["mlp"]["router"])
        by_token = {}
        for t, c in zip(toks, chosen):
            assert by_token.setdefault(t, tuple(sorted(c))) == tuple(sorted(c)), "a token chooses alike wherever it stands"
