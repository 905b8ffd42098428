"""Reselorn on the CPU: its configuration and lowering (which layer keeps the first values and which blend, what the
cache manager makes of the windows, tensors a layer carries without reading them), the rotation's slowed frequencies,
the layer scale folded into a norm's weight, and the plain implementation held against forms that do not share its
loops."""

from __future__ import annotations

import copy
import math

import numpy as np
import pytest
import torch

from miniserve_amd.cache import CacheLayout
from miniserve_amd.config import config_from_dict
from miniserve_amd.config.presets import preset
from miniserve_amd.config.spec import PartSpec
from miniserve_amd.parts.model import CacheSlotNeed, expected_tensors
from miniserve_amd.parts.registry import part_class
from plain import reselorn_plain as R
from plain.model_folder import read_model_folder
from reselorn_models import RESELORN, ROUTER_CHANNELS, make_folder


# ---------------------------------------------------------------- configuration


@pytest.mark.parametrize("name", sorted(RESELORN))
def test_config_reads_back_and_names_its_tensors(name):
    cfg = RESELORN[name][0]
    c = config_from_dict(cfg)
    assert config_from_dict(c.to_dict()).to_dict() == c.to_dict()
    names = expected_tensors(c.to_spec())
    w = cfg["width"]
    assert names["embed"].shape == (cfg["vocab"], w) and names["final.norm"].shape == (w,) and "head" not in names
    blending = False
    for i, layer in enumerate(cfg["layers"]):
        m, mlp = layer["mixer"], layer["mlp"]
        assert names[f"l{i}.mix.q"].shape == (m["heads"] * m["dim"], w)
        assert names[f"l{i}.mix.k"].shape == (m["kv_heads"] * m["dim"], w)
        assert names[f"l{i}.mix.v"].shape == (m["kv_heads"] * m["vdim"], w)
        assert names[f"l{i}.mix.o"].shape == (w, m["heads"] * m["vdim"])
        assert names[f"l{i}.mix.sink"].shape == (m["heads"],)
        assert names[f"l{i}.mix.vmix"].shape == ()
        assert names[f"l{i}.mix.vmix"].optional == (not (m["v_mix"] and blending))  # read by the blending layers alone
        blending = blending or m["v_mix"]
        assert names[f"l{i}.norm1"].shape == names[f"l{i}.ls1"].shape == (w,)
        assert names[f"l{i}.norm2"].optional == names[f"l{i}.ls2"].optional == (not mlp)
        if not mlp:
            assert not any(k.startswith(f"l{i}.mlp.") for k in names)
        elif mlp["kind"] == "dense":
            assert names[f"l{i}.mlp.gate"].shape == names[f"l{i}.mlp.up"].shape == (mlp["ff"], w)
            assert names[f"l{i}.mlp.down"].shape == (w, mlp["ff"])
        else:
            e, f = mlp["router"]["experts"], mlp["expert"]["ff"]
            assert names[f"l{i}.mlp.router"].shape == (e, w) and names[f"l{i}.mlp.router.b"].shape == (e,)
            assert names[f"l{i}.mlp.e{e - 1}.gate"].shape == (f, w) and names[f"l{i}.mlp.e0.down"].shape == (w, f)
            assert f"l{i}.mlp.e{e}.gate" not in names
            assert (f"l{i}.mlp.shared.up" in names) == bool(mlp.get("shared"))
            if mlp.get("shared"):
                assert names[f"l{i}.mlp.shared.down"].shape == (w, mlp["shared"]["ff"])


def test_which_layer_keeps_the_first_values_and_which_blend():
    for name, want in (("rsA", ["first", "blend", None, "blend"]), ("rsB", [None, "first", "blend"]), ("rsC", ["first", "blend", None])):
        spec = config_from_dict(RESELORN[name][0]).to_spec()
        assert [layer.mixer.get("value_blend") for layer in spec.layers] == want, name
        assert [(e.layer, e.cache, e.writes_cache) for e in spec.run_order] == [(i, i, True) for i in range(len(want))]


def test_cache_groups_follow_the_windows_and_the_value_sizes():
    for name in RESELORN:
        cfg = RESELORN[name][0]
        spec = config_from_dict(cfg).to_spec()
        mixers = [part_class("mixer", layer.mixer)(layer.mixer, None) for layer in spec.layers]
        layout = CacheLayout.from_needs([CacheSlotNeed(i, m.kv_need(), m.state_need()) for i, m in enumerate(mixers)])
        assert not layout.states
        for g in layout.groups:
            for s in g.slots:
                m = cfg["layers"][s]["mixer"]
                assert g.window == (m["mask"]["size"] if m.get("mask") else 0)
                planes = {p.name: (p.heads, p.width, p.token_minor) for p in g.planes}
                assert planes == {"k": (m["kv_heads"], m["dim"], False), "v": (m["kv_heads"], m["vdim"], True)}


def test_config_refusals():
    base = RESELORN["rsA"][0]

    def changed(fn):
        c = copy.deepcopy(base)
        fn(c)
        return c

    with pytest.raises(NotImplementedError):
        config_from_dict(changed(lambda c: c["layers"][0].update(type="conv")))
    with pytest.raises(KeyError):
        config_from_dict(changed(lambda c: c["layers"][1]["mixer"].pop("vdim")))
    with pytest.raises(ValueError):
        config_from_dict(changed(lambda c: c["layers"][1]["mixer"].update(kv_heads=4)))  # 6 heads
    with pytest.raises(ValueError):
        config_from_dict(changed(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18)))  # more than dim
    with pytest.raises(ValueError):
        config_from_dict(changed(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7)))
    with pytest.raises(ValueError):
        config_from_dict(changed(lambda c: c["layers"][3]["mixer"].update(vdim=16)))  # cannot be blended with layer 0's
    with pytest.raises(ValueError):
        config_from_dict(changed(lambda c: c["layers"][1]["mlp"]["router"].update(top=6)))  # of 5
    with pytest.raises(KeyError):
        config_from_dict(changed(lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].pop("slow")))
    with pytest.raises(NotImplementedError):
        config_from_dict(changed(lambda c: c["layers"][0]["mlp"].update(kind="routed")))
    assert config_from_dict(preset("reselorn-tiny")).to_spec().architecture == "Reselorn"


def test_the_measured_shapes_are_valid_configurations():
    from miniserve_amd.measurement.designs import SHAPES, reselorn_config

    for name, shape in SHAPES.items():
        spec = config_from_dict(reselorn_config(shape)).to_spec()
        assert len(spec.layers) == shape["layers"], name
        kinds = [layer.feed_forward.kind for layer in spec.layers]
        assert kinds[0] == "gated_mlp" and set(kinds[1:]) == {"moe_mlp"}


def test_tensors_that_nothing_reads_load_and_are_ignored(tmp_path):
    """The first blending layer's blend weight and the second norm and scale of a layer without a feed-forward may be in
    a checkpoint or not; anything else that is unknown is refused."""
    from safetensors.torch import load_file, save_file

    from miniserve_amd.weights.loader import WeightsError, load_weights

    folder = make_folder(tmp_path, "rsA")
    spec = config_from_dict(RESELORN["rsA"][0]).to_spec()
    file = folder / "model.safetensors"
    tensors = load_file(str(file))
    assert "l0.mix.vmix" not in tensors and "l2.mix.vmix" not in tensors and "l3.norm2" not in tensors and "l1.mix.vmix" in tensors
    load_weights(folder, spec, torch.float32, "cpu")
    tensors["l0.mix.vmix"] = torch.tensor(0.5, dtype=torch.bfloat16)
    tensors["l3.norm2"] = torch.zeros(64, dtype=torch.bfloat16)
    tensors["l3.ls2"] = torch.zeros(64, dtype=torch.bfloat16)
    save_file(tensors, str(file))
    load_weights(folder, spec, torch.float32, "cpu")
    tensors["l3.mlp.gate"] = torch.zeros(4, 64, dtype=torch.bfloat16)
    save_file(tensors, str(file))
    with pytest.raises(WeightsError):
        load_weights(folder, spec, torch.float32, "cpu")


# ---------------------------------------------------------------- parts that compute on the host


@pytest.mark.parametrize("dims,base,scaling", [
    (8, 500.0, {"factor": 4.0, "original": 32, "fast": 4.0, "slow": 0.5}),
    (10, 300.0, {"factor": 16.0, "original": 64, "fast": 8.0, "slow": 2.0}),
    (2, 8.0, {"factor": 3.0, "original": 16, "fast": 2.0, "slow": 0.25}),
    (64, 1000.0, {"factor": 2.0, "original": 48, "fast": 4.0, "slow": 0.5}),
    (16, 50.0, {"factor": 5.0, "original": 4096, "fast": 1.0, "slow": 1.0}),   # both ends at one index: the ramp is a step
    (12, 1e6, {"factor": 8.0, "original": 3, "fast": 64.0, "slow": 32.0}),     # both indices below zero: every pair slowed
])
def test_the_rotary_part_slows_frequencies_as_the_plain_form_does(dims, base, scaling):
    spec = PartSpec("rotary", {"dim": dims, "theta": base, "pairing": "halves", "scaling": dict(scaling, kind="turn_ramp")})
    part = part_class("position", spec)(spec, None)
    f, mag = R.slowed_frequencies(dims, base, scaling)
    assert np.allclose(part.inv_freq_host.numpy(), f, rtol=2e-7, atol=0)
    assert math.isclose(part.magnitude, mag, rel_tol=1e-12) and mag == 0.1 * math.log(scaling["factor"]) + 1
    plain = PartSpec("rotary", {"dim": dims, "theta": base})
    assert part_class("position", plain)(plain, None).magnitude == 1.0


def test_slowed_frequencies_by_hand():
    """dims 8, base 500: f = 500^(-i/4). With original 32, the wave of 4 turns lies at index 8 ln(32 / 8 pi) / (2 ln 500)
    = 0.155.. (floor 0) and the wave of half a turn at 1.49.. (ceiling 2): the ramp is 0, 1/2, 1, 1."""
    f, mag = R.slowed_frequencies(8, 500.0, {"factor": 4.0, "original": 32, "fast": 4.0, "slow": 0.5})
    plain = np.array([500.0 ** (-i / 4) for i in range(4)])
    assert np.allclose(f, plain * np.array([1.0, (1 / 4 + 1) / 2, 1 / 4, 1 / 4]))
    assert math.isclose(mag, 0.1 * math.log(4.0) + 1)
    f, mag = R.slowed_frequencies(8, 500.0, None)
    assert np.allclose(f, plain) and mag == 1.0


def test_a_layer_scale_is_folded_into_the_norms_weight():
    spec = PartSpec("rmsnorm", {"width": 6, "eps": 1e-5, "tensor": "n"})
    norm = part_class("norm", spec)(spec, None)
    w = torch.tensor([1.0, 0.5, -2.0, 3.0, 0.25, 1.5], dtype=torch.bfloat16)
    s = torch.tensor([0.5, 2.0, 1.0, 0.0, -4.0, 1.25], dtype=torch.bfloat16)
    norm.bind({"n": w})
    norm.fold_scale(s)
    assert norm.weight.dtype == torch.float32 and torch.equal(norm.weight, w.float() * s.float())
    block = PartSpec("outnorm", {"mixer_norm": spec, "ffn_norm": None, "mixer_scale": "ls", "spare": {"n2": 6}})
    names = part_class("block", block).tensors(block)
    assert names["ls"].shape == (6,) and not names["ls"].optional and names["n2"].optional


# ---------------------------------------------------------------- the plain implementation against other forms


def test_rotation_turns_halves_with_a_magnitude_and_keeps_the_rest():
    rot = {"base": 100.0, "dims": 4, "scaling": {"factor": 4.0, "original": 8, "fast": 2.0, "slow": 0.5}}
    f, mag = R.slowed_frequencies(4, 100.0, rot["scaling"])
    x = (np.arange(2 * 6, dtype=np.float64).reshape(2, 1, 6) + 1)
    out = R.rotate_halves(x, np.array([0, 3]), rot)
    assert np.allclose(out[0, 0, :4], x[0, 0, :4] * mag) and np.allclose(out[:, :, 4:], x[:, :, 4:])
    for i in range(2):
        a = 3 * f[i]
        u, v = x[1, 0, i], x[1, 0, i + 2]
        assert np.allclose([out[1, 0, i], out[1, 0, i + 2]], [mag * (u * math.cos(a) - v * math.sin(a)), mag * (v * math.cos(a) + u * math.sin(a))])
    # scores depend on the distance only
    q, k = np.ones((1, 1, 4)), np.ones((1, 1, 4)) * 0.5
    d1 = R.rotate_halves(q, np.array([9]), rot)[0, 0] @ R.rotate_halves(k, np.array([4]), rot)[0, 0]
    d2 = R.rotate_halves(q, np.array([105]), rot)[0, 0] @ R.rotate_halves(k, np.array([100]), rot)[0, 0]
    assert np.allclose(d1, d2)


def test_softmax_with_a_sink_and_the_window():
    rng = np.random.default_rng(1)
    s = rng.normal(size=(6, 6))
    p = R.sink_softmax(s, R.sliding(6, 3), 0.7)
    for i in range(6):
        js = [j for j in range(6) if 0 <= i - j < 3]
        den = sum(math.exp(s[i, j]) for j in js) + math.exp(0.7)
        for j in range(6):
            assert math.isclose(p[i, j], math.exp(s[i, j]) / den if j in js else 0.0, rel_tol=1e-12, abs_tol=1e-15)
    assert (R.sink_softmax(s, R.sliding(6, 0), -1e9).sum(1) > 1 - 1e-12).all()
    assert R.sliding(5, 0).sum() == 15 and R.sliding(5, 1).sum() == 5


def test_routing_by_hand():
    w = {"router": np.array([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0], [-1.0, 0.0]]), "router.b": np.array([0.0, 0.5, -2.0, 0.0])}
    h = np.array([[2.0, 1.0], [-3.0, 0.0], [0.0, 0.0]])
    chosen, weight = R.route(h, w, 2)
    # logits: [2, 1.5, 1, -2], [-3, .5, -5, 3], [0, .5, -2, 0]; the last row's tie goes to the lower index
    assert chosen.tolist() == [[0, 1], [3, 1], [1, 0]]
    assert np.allclose(weight[0], np.exp([2.0, 1.5]) / np.exp([2.0, 1.5]).sum())
    assert np.allclose(weight.sum(1), 1.0)
    one, full = R.route(h, w, 1)
    assert one.tolist() == [[0], [3], [1]] and np.allclose(full, 1.0)


def test_a_mixture_of_equal_experts_is_one_expert(tmp_path):
    """With every expert the same the softmax's weights sum to one and the mixture is that expert (plus the shared one)."""
    rng = np.random.default_rng(3)
    g, u, d = rng.normal(size=(7, 5)), rng.normal(size=(7, 5)), rng.normal(size=(5, 7))
    w = {"router": rng.normal(size=(4, 5)), "router.b": rng.normal(size=4)}
    for e in range(4):
        w.update({f"e{e}.gate": g, f"e{e}.up": u, f"e{e}.down": d})
    h = rng.normal(size=(9, 5))
    mlp = {"router": {"experts": 4, "top": 3}, "expert": {"ff": 7}}
    want = R.gated_ff(h, {"gate": g, "up": u, "down": d})
    assert np.allclose(R.mixture_ff(h, w, mlp), want)
    w.update({"shared.gate": u, "shared.up": g, "shared.down": d})
    both = R.mixture_ff(h, w, dict(mlp, shared={"ff": 7}))
    assert np.allclose(both, want + R.gated_ff(h, {"gate": u, "up": g, "down": d}))


def test_a_one_layer_model_in_closed_form(tmp_path):
    """One token: the softmax is over one key and the sink, and the rotation at position 0 only multiplies by the magnitude
    (which the division by the root mean square takes out again, but for eps, where the whole head is turned)."""
    cfg = {"architecture": "Reselorn", "vocab": 11, "width": 8, "norm": {"eps": 1e-6}, "layers": [
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 3, "scale": 0.5, "v_mix": True,
                                         "rot": {"base": 10.0, "dims": 4, "scaling": {"factor": 9.0, "original": 8, "fast": 2.0, "slow": 1.0}}},
         "mlp": None}]}
    from miniserve_amd.weights.random_init import Init, write_model_folder

    _, w = read_model_folder(write_model_folder(tmp_path / "one", cfg, 3, Init(0.3, (0.5, 1.5))))
    x = w["embed"][5]
    mag = 0.1 * math.log(9.0) + 1
    q = R.unit_rms(mag * (w["l0.mix.q"] @ x).reshape(2, 4), 1e-6)
    k = R.unit_rms(mag * (w["l0.mix.k"] @ x), 1e-6)
    v = w["l0.mix.v"] @ x
    heads = []
    for a in range(2):
        s = 0.5 * float(q[a] @ k)
        heads.append(v * math.exp(s) / (math.exp(s) + math.exp(float(w["l0.mix.sink"][a]))))
    y = x + R.rms_norm(w["l0.mix.o"] @ np.concatenate(heads), w["l0.norm1"], 1e-6) * w["l0.ls1"]
    want = w["embed"] @ R.rms_norm(y, w["final.norm"], 1e-6)
    assert np.allclose(R.forward(cfg, w, [5])[0], want, rtol=1e-9)


def test_the_test_models_route_by_the_tokens_embedding_alone(tmp_path):
    """What ``make_folder`` promises: the routers read only channels that no sublayer writes, so an expert is chosen by
    the token, whatever came before it and whatever the number format."""
    cfg, w = read_model_folder(make_folder(tmp_path, "rsB"))
    r = ROUTER_CHANNELS
    toks = np.random.default_rng(0).integers(0, cfg["vocab"], size=40)
    _, layers = R.forward(cfg, w, toks, return_layers=True)
    for after in layers:
        assert np.array_equal(after[:, -r:], w["embed"][toks][:, -r:])
    assert not w["l0.mlp.router"][:, :-r].any() and w["l0.mlp.router"][:, -r:].any()
