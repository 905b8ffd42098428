"""Prefill and decode throughput of one architecture beside another of equal size: random weights, layers of the
sizes real models have, the same step function for both. ``bench.py --design kakunex`` (or ``fimolix``, ``reselorn``,
``zigelorn``) prints what this returns.

A *shape* fixes what the two share: width, query and key/value heads of 128 elements, feed-forward width, window,
layers, vocabulary. The Kakunex model of a shape repeats (parallel, parallel, parallel, mlstm): window attention that
keeps the first 4 keys beside a decaying linear attention, and a matrix-memory layer in every fourth place, each
recurrent mixer with as many heads of 128 x 128 as the attention has query heads. The Qwen3 model of the same
shape attends within the same window in every layer.

The Fimolix model of a shape repeats (latent attention, differential attention, differential attention, latent
attention that reads the first one's cache). Its differential attention has half the shape's heads, each with two maps
of 128 and values of 256, so that its four projections have the sizes of the Qwen3 layer's; convolutions of 4 taps. Its
latent attention has the shape's query heads with 128 plain and 64 rotated elements, values of 128 and a latent of 512
per token, inside the shape's window.

The Reselorn model of a shape has the shape's heads of 128 elements (half of them rotated, slowed frequencies), a sink
per head, the shape's window and blended values in every layer; its first layer has the shape's dense feed-forward, the
others a mixture of 32 experts of an eighth of that width, of which a token runs 4, beside a shared expert of half the
width: a token multiplies as much as in the Qwen3 layer, the weights are 4.5 times the layer's.

The Zigelorn model of a shape repeats (wkv, attention, retention, wkv): the attention has the shape's heads of 128 (half
of each rotated, slowed frequencies) inside the shape's window, the retention as many heads of 128 x 128 with rotated
queries and keys, the wkv layers ``width / 64`` heads of 64 x 64 with a decay projection 64 wide. Feed-forwards alternate:
a dense one without a gate, 1.5 times the shape's width (as many multiplications as the gated one of the shape), and a
mixture of 28 experts of a quarter of that beside 4 identity experts, 8 groups of which 4 are kept, 4 chosen. It is
measured beside the Kakunex model of the shape, the other design of windowed attention and linear recurrences."""

from __future__ import annotations

import statistics
import time

SHAPES = {
    # name: width, heads, kv_heads, feed-forward, window, layers, vocabulary
    "w1024": dict(width=1024, heads=8, kv_heads=4, ff=3072, window=1024, layers=8, vocab=32768),
    "w2048": dict(width=2048, heads=16, kv_heads=4, ff=8192, window=2048, layers=8, vocab=32768),
    "w4096": dict(width=4096, heads=32, kv_heads=8, ff=12288, window=2048, layers=4, vocab=32768),
}
HEAD = 128
KEEP_FIRST = 4


def kakunex_config(s: dict) -> dict:
    decays = [1.0 - 2.0 ** -(3 + 7 * i / max(1, s["heads"] - 1)) for i in range(s["heads"])]
    left = {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": HEAD, "vdim": HEAD, "scale": HEAD ** -0.5,
            "rot": {"base": 5e5, "dims": HEAD // 2, "scaling": {"factor": 4.0, "low": 1.0, "high": 8.0, "original": 4096}},
            "mask": {"size": s["window"], "keep_first": KEEP_FIRST}}
    right = {"heads": s["heads"], "dim": HEAD, "vdim": HEAD, "decay": decays}
    mlp = {"kind": "dense", "ff": s["ff"], "limit": 7.0}
    layers = []
    for i in range(s["layers"]):
        if i % 4 == 3:
            layers.append({"type": "mlstm", "mixer": {"heads": s["heads"], "dim": HEAD, "vdim": HEAD, "gate_cap": 10.0}, "mlp": mlp})
        else:
            layers.append({"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp})
    return {"architecture": "Kakunex", "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-6}, "logit_scale": 1.0,
            "layers": layers}


def qwen3_config(s: dict) -> dict:
    return {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "hidden_act": "silu", "num_hidden_layers": s["layers"],
            "hidden_size": s["width"], "num_attention_heads": s["heads"], "num_key_value_heads": s["kv_heads"], "head_dim": HEAD,
            "intermediate_size": s["ff"], "vocab_size": s["vocab"], "rope_theta": 1e6, "rms_norm_eps": 1e-6,
            "tie_word_embeddings": True, "max_position_embeddings": 40960, "sliding_window": s["window"],
            "layer_types": ["sliding_attention"] * s["layers"]}


LATENT, ROTATED = 512, 64


def fimolix_config(s: dict) -> dict:
    mlp = {"kind": "dense", "ff": s["ff"]}
    maps = {"heads": s["heads"] // 2, "kv_heads": max(1, s["kv_heads"] // 2), "dim": HEAD, "vdim": 2 * HEAD, "scale": HEAD ** -0.5,
            "softcap": 30.0, "conv": 4, "diff": 0.4}
    latent = {"heads": s["heads"], "dim": HEAD, "rot_dim": ROTATED, "vdim": HEAD, "kv_rank": LATENT, "scale": (HEAD + ROTATED) ** -0.5,
              "rot": {"base": 1e4, "dims": ROTATED}, "mask": {"size": s["window"]}}
    layers = []
    for i in range(s["layers"]):
        if i % 4 in (1, 2):
            layers.append({"type": "attention", "mixer": dict(maps), "mlp": mlp})
        else:
            layers.append({"type": "latent_attention", "mixer": dict(latent, **({"kv_from": i - 3} if i % 4 == 3 else {})), "mlp": mlp})
    return {"architecture": "Fimolix", "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-6}, "layers": layers}


EXPERTS, CHOSEN = 32, 4


def reselorn_config(s: dict) -> dict:
    mixer = {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": HEAD, "vdim": HEAD, "scale": HEAD ** -0.5, "v_mix": True,
             "rot": {"base": 1.5e5, "dims": HEAD // 2, "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}},
             "mask": {"size": s["window"]}}
    mixture = {"kind": "moe", "router": {"experts": EXPERTS, "top": CHOSEN}, "expert": {"ff": s["ff"] // 8}, "shared": {"ff": s["ff"] // 2}}
    layers = [{"type": "attention", "mixer": dict(mixer), "mlp": {"kind": "dense", "ff": s["ff"]} if i == 0 else mixture}
              for i in range(s["layers"])]
    return {"architecture": "Reselorn", "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-6}, "layers": layers}


def zigelorn_config(s: dict) -> dict:
    rot = {"base": 1e6, "dims": HEAD // 2, "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}}
    attention = {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": HEAD, "vdim": HEAD, "scale": HEAD ** -0.5, "rot": rot,
                 "mask": {"size": s["window"]}}
    decays = [1.0 - 2.0 ** -(5 + 6 * i / max(1, s["heads"] - 1)) for i in range(s["heads"])]
    retention = {"heads": s["heads"], "dim": HEAD, "vdim": HEAD, "decay": decays, "rot": {"base": 1e6, "dims": HEAD}}
    wkv = {"heads": s["width"] // 64, "dim": 64, "rank": 64}
    ff = s["ff"] * 3 // 2
    dense = {"kind": "dense", "ff": ff}
    mixture = {"kind": "moe", "router": {"experts": 28, "identity": 4, "top": 4, "groups": {"count": 8, "keep": 4}}, "expert": {"ff": ff // 4}}
    kinds = (("wkv", wkv, dense), ("attention", attention, mixture), ("retention", retention, dense), ("wkv", wkv, mixture))
    layers = [{"type": kinds[i % 4][0], "mixer": dict(kinds[i % 4][1]), "mlp": dict(kinds[i % 4][2])} for i in range(s["layers"])]
    return {"architecture": "Zigelorn", "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-6}, "layers": layers}


DESIGNS = {"kakunex": kakunex_config, "fimolix": fimolix_config, "reselorn": reselorn_config, "zigelorn": zigelorn_config,
           "qwen3": qwen3_config}
BESIDE = {"zigelorn": "kakunex"}  # the model a design is measured beside (default: qwen3)


def measure(config: dict, dtype: str, prefill_tokens: int, batch: int, context: int, steps: int, warmup: int, say=lambda m: None) -> dict:
    """Tokens per second of one ``prefill_tokens``-token prompt in one step (median of three after one untimed), and of
    ``steps`` decode steps of ``batch`` requests that each hold ``context`` tokens (replayed as captured graphs, after
    ``warmup`` untimed steps)."""
    import torch

    from ..engine.batch import StepRow
    from ..engine.runner import ModelRunner
    from ..loading import random_model
    from .markers import measured_region

    model = random_model(config, seed=0, dtype=dtype)
    vocab = model.vocab_size
    gen = torch.Generator().manual_seed(0)

    def ids(n):
        return torch.randint(0, vocab, (n,), generator=gen).tolist()

    runner = ModelRunner(model, kv_pool_tokens=max(2 * prefill_tokens, batch * (context + 64)) + 64, max_running=batch,
                         decode_graph=True)
    times = []
    for i in range(4):
        rc = runner.acquire()
        toks = ids(prefill_tokens)
        torch.cuda.synchronize()
        with measured_region("prefill" if i else "prefill (untimed)"):
            t0 = time.perf_counter()
            runner.step([StepRow(rc, toks, [prefill_tokens - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        runner.release(rc)
    prefill_s = statistics.median(times[1:])
    say(f"  prefill of {prefill_tokens} tokens: {prefill_s * 1e3:.2f} ms")
    handles = [runner.acquire() for _ in range(batch)]
    first = context - warmup - steps
    for rc in handles:
        for at in range(0, first, 2048):
            runner.step([StepRow(rc, ids(min(2048, first - at)), [])])
    for _ in range(warmup):
        runner.step([StepRow(rc, ids(1), [0]) for rc in handles])
    torch.cuda.synchronize()
    with measured_region("decode"):
        t0 = time.perf_counter()
        for _ in range(steps):
            runner.step([StepRow(rc, ids(1), [0]) for rc in handles])
        torch.cuda.synchronize()
        decode_s = (time.perf_counter() - t0) / steps
    say(f"  decode step of {batch} rows at context {context}: {decode_s * 1e3:.3f} ms")
    for rc in handles:
        runner.release(rc)
    out = {"prefill_tok_s": round(prefill_tokens / prefill_s, 1), "prefill_ms": round(prefill_s * 1e3, 3),
           "prefill_tflops": round(model.step_flops([(prefill_tokens, 0)]) / prefill_s / 1e12, 1),
           "decode_tok_s": round(batch / decode_s, 1), "decode_ms_per_step": round(decode_s * 1e3, 4),
           "decode_weight_gbs": round(model.decode_read_bytes(batch) / decode_s / 1e9, 1),
           "weights_gb": round(model.decode_read_bytes(batch) / 1e9, 3)}
    del runner, model
    torch.cuda.empty_cache()
    return out


def compare(design: str, shapes=None, dtype: str = "bfloat16", prefill_tokens: int = 2048, batch: int = 8, context: int = 2048,
            steps: int = 32, warmup: int = 8, beside: str | None = None, say=lambda m: None) -> dict:
    """``{shape: {design: figures, beside: figures}}`` for the named shapes (all by default)."""
    beside = beside or BESIDE.get(design, "qwen3")
    out = {}
    for name in shapes or sorted(SHAPES):
        s = SHAPES[name]
        out[name] = {"shape": dict(s, head=HEAD, keep_first=KEEP_FIRST)}
        for which in (design, beside):
            say(f"{name}: {which}")
            out[name][which] = measure(DESIGNS[which](s), dtype, prefill_tokens, batch, context, steps, warmup, say)
    return out
