"""Named ``config.json`` dictionaries: two tiny shapes that differ in every size and option, one
tiny windowed shape, the three benchmark shapes, one tiny Kakunex and one tiny Fimolix model (random weights; no checkpoint is fetched).

The reference names models by size and maps them to pinned downloads
(miniserve/model/weights.py:24-29); without a network the names map to shapes instead.
"""

from __future__ import annotations

import copy


def _qwen3(**kw) -> dict:
    base = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "hidden_act": "silu"}
    base.update(kw)
    return base


PRESETS: dict[str, dict] = {
    "tinyA": _qwen3(
        num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
        intermediate_size=128, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6,
        tie_word_embeddings=True, max_position_embeddings=128,
    ),
    "tinyB": _qwen3(
        num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=1, head_dim=32,
        intermediate_size=224, vocab_size=379, rope_theta=1e6, rms_norm_eps=1e-5,
        tie_word_embeddings=False, max_position_embeddings=256,
    ),
    "tinyC": _qwen3(
        num_hidden_layers=4, hidden_size=80, num_attention_heads=3, num_key_value_heads=3, head_dim=48,
        intermediate_size=176, vocab_size=517, rope_theta=50000.0, rms_norm_eps=3e-6,
        tie_word_embeddings=False, max_position_embeddings=512, sliding_window=24,
        layer_types=["sliding_attention", "full_attention", "sliding_attention", "sliding_attention"],
    ),
    # Head sizes 64 and 128 with 16-token pages: the shapes the matrix-core attention kernels take.
    "tinyD": _qwen3(
        num_hidden_layers=2, hidden_size=128, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
        intermediate_size=192, vocab_size=300, rope_theta=10000.0, rms_norm_eps=1e-6,
        tie_word_embeddings=True, max_position_embeddings=2048,
    ),
    "tinyE": _qwen3(
        num_hidden_layers=3, hidden_size=160, num_attention_heads=4, num_key_value_heads=1, head_dim=128,
        intermediate_size=288, vocab_size=411, rope_theta=1e6, rms_norm_eps=1e-5,
        tie_word_embeddings=False, max_position_embeddings=4096, sliding_window=100,
        layer_types=["full_attention", "sliding_attention", "full_attention"],
    ),
    "0.6B": _qwen3(
        num_hidden_layers=28, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
        intermediate_size=3072, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
        tie_word_embeddings=True, max_position_embeddings=40960,
    ),
    "8B": _qwen3(
        num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
        intermediate_size=12288, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
        tie_word_embeddings=False, max_position_embeddings=40960,
    ),
    "32B": _qwen3(
        num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
        intermediate_size=25600, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
        tie_word_embeddings=False, max_position_embeddings=40960,
    ),
}


def _kakunex_tiny() -> dict:
    """Three layers that hold every part of the architecture once: windowed attention that keeps the first keys beside
    a decaying linear attention, an mLSTM layer without a feed-forward, and an attention that rotates the whole head."""
    bands = {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 64}

    def pair(heads, kv_heads, dim, vdim, rot, mask, lin_heads, lin_dim, lin_vdim, decay, ff):
        left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "rot": rot, "mask": mask}
        right = {"heads": lin_heads, "dim": lin_dim, "vdim": lin_vdim, "decay": decay}
        return {"type": "parallel", "mixer": {"left": left, "right": right},
                "mlp": {"kind": "dense", "ff": ff, "limit": 4.0} if ff else None}

    return {
        "architecture": "Kakunex", "vocab": 311, "width": 96, "norm": {"eps": 1e-5}, "logit_scale": 0.5,
        "layers": [
            pair(4, 2, 32, 16, {"base": 1000.0, "dims": 16, "scaling": bands}, {"size": 24, "keep_first": 6}, 3, 16, 32,
                 [0.7, 0.95, 0.999], 160),
            {"type": "mlstm", "mixer": {"heads": 2, "dim": 24, "vdim": 48, "gate_cap": 8.0}, "mlp": None},
            pair(3, 3, 16, 32, {"base": 1000.0, "dims": 16}, {"size": 40, "keep_first": 0}, 2, 8, 48, [0.9, 0.99], 128),
        ],
    }


PRESETS["kakunex-tiny"] = _kakunex_tiny()


def _fimolix_tiny() -> dict:
    """Four layers that hold every part of the architecture once: a latent attention with a window, a differential
    attention with a convolution of three taps, a second latent attention that reads the first one's cache through a
    wider window and has no feed-forward, and a differential attention whose heads share one key/value head."""
    rot = {"base": 5000.0, "dims": 8}

    def latent(heads, dim, vdim, size, ff, kv_from=None):
        m = {"heads": heads, "dim": dim, "rot_dim": 8, "vdim": vdim, "kv_rank": 40, "scale": (dim + 8) ** -0.5, "rot": rot,
             "mask": {"size": size}}
        if kv_from is not None:
            m["kv_from"] = kv_from
        return {"type": "latent_attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}

    def attention(heads, kv_heads, dim, vdim, conv, diff, ff):
        m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "softcap": 20.0, "conv": conv,
             "diff": diff}
        return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}

    return {
        "architecture": "Fimolix", "vocab": 311, "width": 96, "norm": {"eps": 1e-5},
        "layers": [latent(4, 16, 24, 24, 160), attention(4, 2, 16, 32, 3, 0.4, 128), latent(2, 24, 16, 56, None, kv_from=0),
                   attention(3, 1, 32, 16, 4, 0.6, 160)],
    }


PRESETS["fimolix-tiny"] = _fimolix_tiny()


def _reselorn_tiny() -> dict:
    """Four layers that hold every part of the architecture once: a dense layer that makes the first values, a mixture
    with a shared expert whose values are blended, a layer that neither blends nor has a feed-forward and sees every
    earlier token, and a mixture without a shared expert behind a rotation that is not slowed down."""
    slowed = {"base": 3000.0, "dims": 12, "scaling": {"factor": 8.0, "original": 48, "fast": 6.0, "slow": 0.5}}

    def attention(heads, kv_heads, dim, rot, size, v_mix, mlp):
        m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": 24, "scale": dim ** -0.5, "rot": rot, "v_mix": v_mix}
        if size:
            m["mask"] = {"size": size}
        return {"type": "attention", "mixer": m, "mlp": mlp}

    def moe(experts, top, ff, shared):
        out = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
        if shared:
            out["shared"] = {"ff": shared}
        return out

    return {
        "architecture": "Reselorn", "vocab": 311, "width": 96, "norm": {"eps": 1e-5},
        "layers": [attention(4, 2, 32, slowed, 24, True, {"kind": "dense", "ff": 160}),
                   attention(6, 2, 16, slowed, 40, True, moe(6, 2, 48, 80)),
                   attention(2, 1, 48, {"base": 100.0, "dims": 48}, 0, False, None),
                   attention(4, 2, 32, {"base": 3000.0, "dims": 12}, 24, True, moe(5, 3, 32, None))],
    }


PRESETS["reselorn-tiny"] = _reselorn_tiny()


def _zigelorn_tiny() -> dict:
    """Six layers that hold every part of the architecture once: the three mixers, a dense feed-forward, a mixture with
    identity experts and groups, a layer without a feed-forward, and a layer that runs another's weights over a state of its own."""
    slowed = {"base": 3000.0, "dims": 12, "scaling": {"factor": 8.0, "original": 48, "fast": 6.0, "slow": 0.5}}
    attention = {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 24, "scale": 24 ** -0.5, "rot": slowed,
                                                "mask": {"size": 24}},
                 "mlp": {"kind": "moe", "router": {"experts": 6, "identity": 2, "top": 3, "groups": {"count": 4, "keep": 2}},
                         "expert": {"ff": 48}}}
    wkv = {"type": "wkv", "mixer": {"heads": 3, "dim": 32, "rank": 12}, "mlp": {"kind": "dense", "ff": 160}}
    retention = {"type": "retention", "mixer": {"heads": 3, "dim": 16, "vdim": 32, "decay": [0.9, 0.97, 0.995],
                                                "rot": {"base": 100.0, "dims": 16}}, "mlp": None}
    return {
        "architecture": "Zigelorn", "vocab": 311, "width": 96, "norm": {"eps": 1e-5},
        "layers": [wkv, attention, retention, dict(copy.deepcopy(attention), weights_of=1), dict(copy.deepcopy(wkv), weights_of=0),
                   {"type": "retention", "mixer": {"heads": 2, "dim": 8, "vdim": 8, "decay": [0.5, 1.0]}, "mlp": {"kind": "dense", "ff": 64}}],
    }


PRESETS["zigelorn-tiny"] = _zigelorn_tiny()


def preset(name: str) -> dict:
    try:
        return copy.deepcopy(PRESETS[name])
    except KeyError:
        raise ValueError(f"unknown preset {name!r}, expected one of {sorted(PRESETS)}") from None
