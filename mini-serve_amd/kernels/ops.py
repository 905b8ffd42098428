"""The kernel library as Python calls: every function checks shapes, dtypes and contiguity on the
host, then launches hand-written HIP kernels on torch's current stream. There is no fallback:
without a GPU or without the built library these calls raise.

Tensors are torch tensors used as plain device buffers; no torch operator computes anything here.
"""

from __future__ import annotations

import ctypes

import torch

from . import build

_lib = None

F32, BF16, I32 = torch.float32, torch.bfloat16, torch.int32
_c_void, _c_int, _c_float, _c_ll = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_longlong

_ERRORS = {1: "bad argument", 2: "unsupported size", 3: "kernel launch failed"}

_SIGNATURES = {
    "ms_embed": [_c_void, _c_void, _c_int, _c_void, _c_int, _c_int, _c_void],
    "ms_feed_tokens": [_c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_void],
    "ms_rmsnorm": [_c_void, _c_void, _c_int, _c_void, _c_int, _c_void, _c_int, _c_int, _c_float, _c_void, _c_int, _c_ll, _c_void],
    "ms_act_mul": [_c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_void],
    "ms_act_mul_parts": [_c_void, _c_int, _c_ll, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_void],
    "ms_layernorm": [_c_void, _c_void, _c_void, _c_int, _c_void, _c_int, _c_void, _c_int, _c_int, _c_float, _c_void],
    "ms_group_rmsnorm_gate": [_c_void, _c_void, _c_int, _c_void, _c_int, _c_void, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void],
    "ms_normed_mean_add": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_void],
    "ms_normed_add_pending": [_c_void, _c_void, _c_void, _c_int, _c_ll, _c_void, _c_int, _c_int, _c_int, _c_float, _c_void, _c_int,
                              _c_void],
    "ms_scale": [_c_void, _c_ll, _c_float, _c_void],
    "ms_qkv_norm_rope_store": [_c_void, _c_int, _c_void, _c_int, _c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_float, _c_void,
                               _c_int, _c_int, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_gated_recurrence": [_c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                            _c_float, _c_void, _c_void, _c_void, _c_int, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                            _c_int, _c_void, _c_int, _c_void, _c_void],
    "ms_rotate_columns": [_c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void, _c_int, _c_int, _c_float, _c_void],
    "ms_token_shift_mix": [_c_void, _c_void, _c_void, _c_int, _c_void, _c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_void],
    "ms_neg_exp_bias": [_c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_wkv_chunked": [_c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void, _c_int, _c_void, _c_void, _c_void, _c_void, _c_void,
                       _c_void, _c_int, _c_int, _c_void, _c_void, _c_void],
    "ms_wkv_chunk_tokens": [],
    "ms_wkv_chunk_max_dim": [],
    "ms_gated_recurrence_chunked": [_c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                    _c_float, _c_float, _c_void, _c_void, _c_void, _c_int, _c_void, _c_void, _c_void, _c_void, _c_void,
                                    _c_void, _c_void, _c_int, _c_int, _c_void, _c_void, _c_void, _c_void],
    "ms_gated_recurrence_chunk_tokens": [],
    "ms_gated_recurrence_chunk_max_dim": [],
    "ms_gemm_bf16_gated": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_cast": [_c_void, _c_int, _c_void, _c_int, _c_ll, _c_void],
    "ms_rope_table": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_float, _c_void],
    "ms_qk_norm_rope_store": [_c_void, _c_void, _c_int, _c_ll, _c_void, _c_int, _c_int, _c_void, _c_void, _c_void,
                              _c_int, _c_float, _c_void, _c_int, _c_int, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int,
                              _c_void],
    "ms_gemm_f32": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_gemm_bf16": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_gemm_bf16_tile_splits": [_c_int, _c_int, _c_int],
    "ms_gemm_bf16_tile_shape": [_c_int, _c_int, _c_int, _c_int, _c_int, _c_int],
    "ms_gemm_bf16_small": [_c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_gemm_bf16_small_splits": [_c_int, _c_int, _c_int],
    "ms_gemm_bf16_small_tile_cols": [_c_int, _c_int],
    "ms_splitk_reduce": [_c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_paged_attention_generic": [_c_void, _c_int, _c_void, _c_void, _c_int, _c_void, _c_int, _c_void, _c_void, _c_void,
                                   _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_int,
                                   _c_float, _c_void, _c_int, _c_int, _c_int, _c_void],
    "ms_conv_norm_store": [_c_void, _c_int, _c_void, _c_int, _c_int, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                           _c_void, _c_float, _c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                           _c_int, _c_int, _c_int, _c_void],
    "ms_map_difference_norm": [_c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_float, _c_void],
    "ms_latent_prepare": [_c_void, _c_int, _c_int, _c_int, _c_void, _c_int, _c_int, _c_void, _c_int, _c_float, _c_void, _c_void,
                          _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_paged_attention_tiled_mfma_wide": [_c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_void, _c_void, _c_int, _c_void, _c_void,
                                           _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_float,
                                           _c_void, _c_int, _c_int, _c_void, _c_void, _c_void],
    "ms_paged_attention_tiled_mfma_wide_chunk": [_c_int, _c_int, _c_int, _c_int, _c_int],
    "ms_head_gemm_bf16": [_c_void, _c_int, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void, _c_int,
                          _c_int, _c_void],
    "ms_head_gate": [_c_void, _c_int, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_activate": [_c_void, _c_void, _c_int, _c_ll, _c_int, _c_void],
    "ms_paged_attention_tiled": [_c_void, _c_int, _c_void, _c_void, _c_int, _c_void, _c_int, _c_void, _c_void, _c_int, _c_void, _c_void,
                                 _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_void],
    "ms_paged_attention_tiled_tokens": [_c_int, _c_int, _c_int],
    "ms_paged_attention_tiled_mfma": [_c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_void, _c_void, _c_int, _c_void, _c_void,
                                      _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_void],
    "ms_paged_attention_tiled_mfma_ok": [_c_int, _c_int, _c_int],
    "ms_attention_decode_bf16": [_c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_void, _c_void, _c_void, _c_void,
                                 _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void],
    "ms_attention_decode_fused_bf16": [_c_void, _c_int, _c_ll, _c_void, _c_void, _c_float, _c_void, _c_int, _c_int, _c_void, _c_void,
                                       _c_void, _c_int, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_int, _c_int,
                                       _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_void],
    "ms_attention_merge_project": [_c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_attention_merge_project_splits": [_c_int, _c_int, _c_int, _c_int, _c_int],
    "ms_attention_prefill_bf16": [_c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_void, _c_void, _c_int, _c_int,
                                  _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void],
    "ms_attention_prefill_parts_bf16": [_c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_void, _c_int, _c_int, _c_void,
                                        _c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_float,
                                        _c_void],
    "ms_attention_prefill_tile_tokens": [_c_int, _c_int],
    "ms_sample_rows": [_c_void, _c_int, _c_int, _c_ll, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void],
    "ms_sample_scratch_bytes": [_c_int],
    "ms_sample_rows_static": [_c_void, _c_int, _c_int, _c_ll, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void],
    "ms_sample_rows_static_max_rows": [],
    "ms_head_prepare_store": [_c_void, _c_int, _c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_int, _c_float, _c_void, _c_int,
                              _c_int, _c_void, _c_int, _c_float, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                              _c_void],
    "ms_moe_route": [_c_void, _c_int, _c_int, _c_ll, _c_void, _c_int, _c_int, _c_int, _c_int, _c_void, _c_void, _c_void],
    "ms_moe_route_scored": [_c_void, _c_int, _c_int, _c_ll, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void, _c_void, _c_void],
    "ms_moe_plan": [_c_void, _c_int, _c_int, _c_int, _c_int, _c_void, _c_void, _c_void, _c_void, _c_void],
    "ms_moe_gemm": [_c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_int, _c_void, _c_void, _c_void, _c_void, _c_void,
                    _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_moe_combine": [_c_void, _c_void, _c_int, _c_int, _c_int, _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_void],
    "ms_measure_read": [_c_void, _c_ll, _c_int, _c_void, _c_void],
    "ms_measure_copy": [_c_void, _c_void, _c_ll, _c_int, _c_void],
}


class KernelLibraryMissing(RuntimeError):
    pass


def library():
    """The loaded kernel library; built first if no build of the current sources exists."""
    global _lib
    if _lib is None:
        if not torch.cuda.is_available():
            raise KernelLibraryMissing("no GPU is visible: the engine runs on HIP kernels only and has no CPU fallback")
        try:
            path = build.build_kernels()
            lib = ctypes.CDLL(str(path))
        except Exception as e:  # noqa: BLE001
            raise KernelLibraryMissing(f"the HIP kernel library could not be built or loaded: {e}") from e
        for name, args in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = _c_int
        _lib = lib
    return _lib


def library_path() -> str:
    return str(build.build_kernels())


_pinned_stream: int | None = None


def _stream() -> int:
    return _pinned_stream if _pinned_stream is not None else torch.cuda.current_stream().cuda_stream


class stream_scope:
    """Looks the current HIP stream up once for all kernel launches inside the ``with`` block (the
    lookup costs several microseconds, a model pass makes hundreds). The stream must not be switched
    inside the block."""

    def __enter__(self):
        global _pinned_stream
        self._before = _pinned_stream
        _pinned_stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        global _pinned_stream
        _pinned_stream = self._before
        return False


def _check(code: int, what: str) -> None:
    if code:
        raise RuntimeError(f"{what}: {_ERRORS.get(code, code)}")


def _dev(t: torch.Tensor, name: str, dtypes, ndim: int | None = None) -> None:
    """A contiguous tensor on the GPU of one of ``dtypes`` (and of ``ndim`` dimensions). A model pass
    makes hundreds of these checks: what is right passes in three calls; what is wrong is looked at
    again, slowly, for the message."""
    try:
        if t.is_cuda and t.is_contiguous() and (t.dtype is dtypes or t.dtype in dtypes) and (ndim is None or t.dim() == ndim):
            return
    except (AttributeError, TypeError):
        pass
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError(f"{name} must be a tensor on the GPU")
    if t.dtype not in (dtypes if isinstance(dtypes, tuple) else (dtypes,)):
        raise TypeError(f"{name} has dtype {t.dtype}, expected {dtypes}")
    if ndim is not None and t.dim() != ndim:
        raise ValueError(f"{name} has {t.dim()} dimensions, expected {ndim}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def _ptr(t) -> int | None:
    return None if t is None else t.data_ptr()


class SplitSum:
    """A matrix that exists only as partial sums: its value is ``parts.sum(0)`` (float32
    ``[splits, M, N]``, to be added in ascending split order). The small-M matrix product leaves its
    result in this form so that the kernel that consumes it does the summing and no kernel of its own
    is spent on it. ``accumulate`` marks a sum that still has to be added to the residual stream."""

    __slots__ = ("parts",)

    def __init__(self, parts: torch.Tensor):
        self.parts = parts

    @property
    def shape(self):
        return tuple(self.parts.shape[1:])

    @property
    def splits(self) -> int:
        return self.parts.shape[0]

    @property
    def stride(self) -> int:
        return self.parts.shape[1] * self.parts.shape[2]


def _check_split(v: SplitSum, name: str, shape) -> None:
    _dev(v.parts, name, F32, 3)
    if v.shape != tuple(shape):
        raise ValueError(f"{name} holds partial sums of a {v.shape} matrix, expected {tuple(shape)}")


# ------------------------------------------------------------------------------------- elementwise


def embed(token_ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """``float32 [T, width]`` rows of ``table`` (float32 or bfloat16). Ids must be in range (the
    caller checks them on the host before they are uploaded)."""
    _dev(token_ids, "token_ids", I32, 1)
    _dev(table, "table", (F32, BF16), 2)
    out = torch.empty((token_ids.shape[0], table.shape[1]), dtype=F32, device=table.device)
    _check(library().ms_embed(token_ids.data_ptr(), table.data_ptr(), int(table.dtype == BF16), out.data_ptr(),
                              token_ids.shape[0], table.shape[1], _stream()), "embed")
    return out


def feed_tokens(token_ids: torch.Tensor, row_start: torch.Tensor | None, feed: torch.Tensor, source: torch.Tensor) -> None:
    """In place: the last token of row ``i`` of ``token_ids`` becomes ``source[feed[i]]`` where
    ``feed[i] >= 0``. ``row_start``: ``rows + 1`` offsets of the rows in ``token_ids`` (None: one token
    per row). For tokens that were sampled on the device and not yet read back."""
    _dev(token_ids, "token_ids", I32, 1)
    _dev(feed, "feed", I32, 1)
    _dev(source, "source", I32, 1)
    rows = feed.shape[0]
    if row_start is not None:
        _dev(row_start, "row_start", I32, 1)
        if row_start.shape[0] != rows + 1:
            raise ValueError("row_start must hold one offset more than there are rows")
    elif token_ids.shape[0] < rows:
        raise ValueError("fewer tokens than rows")
    _check(library().ms_feed_tokens(token_ids.data_ptr(), _ptr(row_start), feed.data_ptr(), source.data_ptr(), rows,
                                    source.shape[0], _stream()), "feed_tokens")


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype, rows: torch.Tensor | None = None,
            add: SplitSum | None = None) -> torch.Tensor:
    """RMSNorm of the float32 rows of ``x`` (all, or those named by ``rows``). ``add``: a pending sum that
    is added to the rows first; without ``rows`` also into ``x`` itself (in place), with ``rows`` (which
    may name a row twice) ``x`` is left unchanged."""
    _dev(x, "x", F32, 2)
    _dev(weight, "weight", (F32, BF16), 1)
    if weight.shape[0] != x.shape[1]:
        raise ValueError(f"norm weight has {weight.shape[0]} elements for width {x.shape[1]}")
    if out_dtype not in (F32, BF16):
        raise TypeError(f"unsupported output dtype {out_dtype}")
    n = x.shape[0]
    if rows is not None:
        _dev(rows, "rows", I32, 1)
        n = rows.shape[0]
    parts, splits, stride = None, 0, 0
    if add is not None:
        _check_split(add, "add", x.shape)
        parts, splits, stride = add.parts.data_ptr(), add.splits, add.stride
    out = torch.empty((n, x.shape[1]), dtype=out_dtype, device=x.device)
    _check(library().ms_rmsnorm(x.data_ptr(), weight.data_ptr(), int(weight.dtype == BF16), out.data_ptr(),
                                int(out_dtype == BF16), _ptr(rows), n, x.shape[1], float(eps), parts, splits, stride,
                                _stream()), "rmsnorm")
    return out


GATE_BLOCK = 16  # rows per run of gate / up rows in an interleaved gate-up weight


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``[2 I, K]`` with alternating runs of ``GATE_BLOCK`` gate rows and ``GATE_BLOCK`` up rows: the
    order in which the matrix kernels hold gate and up of one output in one lane. ``I`` must be a
    multiple of ``GATE_BLOCK``."""
    i, k = gate.shape
    if up.shape != gate.shape or i % GATE_BLOCK:
        raise ValueError(f"gate {tuple(gate.shape)} and up {tuple(up.shape)} cannot be interleaved in runs of {GATE_BLOCK}")
    both = torch.stack((gate.view(i // GATE_BLOCK, GATE_BLOCK, k), up.view(i // GATE_BLOCK, GATE_BLOCK, k)), dim=1)
    return both.reshape(2 * i, k).contiguous()


# Activations of the gated feed-forward and the numbers the kernels know them by (MS_ACT_* in csrc/common.h):
# silu(x) = x sigmoid(x); gelu_tanh(x) = x / 2 (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3))).
# swiglu_clamped(gate, up) = g sigmoid(1.702 g) (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit): not of
# the form act(gate) * up, it takes ``limit`` along and runs in the activation kernels (no matrix kernel's epilogue knows it).
ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "swiglu_clamped": 2, "relu_squared": 3, "tanh": 4}
ACTIVATIONS_UNGATED_ONLY = {"relu_squared", "tanh"}  # no kernel finishes act(gate) * up with these
ACTIVATIONS_WITH_LIMIT = {"swiglu_clamped"}


def _activation(name: str, limit: float | None = None, gated: bool = True) -> int:
    try:
        act = ACTIVATIONS[name]
    except KeyError:
        raise NotImplementedError(f"activation {name!r}: the kernels know {sorted(ACTIVATIONS)}") from None
    if gated and name in ACTIVATIONS_UNGATED_ONLY:
        raise NotImplementedError(f"activation {name!r} has no gated form act(gate) * up here")
    if name in ACTIVATIONS_WITH_LIMIT and not (limit is not None and limit > 0):
        raise ValueError(f"activation {name!r} needs a positive limit, got {limit!r}")
    return act


def act_mul(gu, activation: str = "silu", out_dtype=None, block: int = 0, limit: float | None = None) -> torch.Tensor:
    """``act(gate) * up`` (or what ``activation`` makes of gate and up) for ``gu [T, 2 I]``, a tensor or a
    ``SplitSum`` (then ``out_dtype`` names the
    result's dtype). ``block == 0``: the row holds the ``I`` gates, then the ``I`` ups; ``block > 0``:
    alternating runs of ``block`` gates and ``block`` ups (see ``interleave_gate_up``)."""
    act = _activation(activation, limit)
    limit = float(limit or 0.0)
    if isinstance(gu, SplitSum):
        _dev(gu.parts, "gu", F32, 3)
        t, width = gu.shape
        if width % 2 or out_dtype not in (F32, BF16) or (block and (width // 2) % block):
            raise ValueError("gate/up partial sums need an even width (whole runs) and an output dtype")
        out = torch.empty((t, width // 2), dtype=out_dtype, device=gu.parts.device)
        for t0 in range(0, t, 32768):
            n = min(32768, t - t0)
            _check(library().ms_act_mul_parts(gu.parts[:, t0:].data_ptr(), gu.splits, gu.stride, out[t0:].data_ptr(),
                                              int(out_dtype == BF16), n, width // 2, int(block), act, limit, _stream()), "act_mul")
        return out
    _dev(gu, "gu", (F32, BF16), 2)
    if gu.shape[1] % 2 or (block and (gu.shape[1] // 2) % block):
        raise ValueError("gate/up buffer needs an even width (whole runs)")
    inter = gu.shape[1] // 2
    out = torch.empty((gu.shape[0], inter), dtype=gu.dtype, device=gu.device)
    # grid.y carries the token index: split very long batches
    for t0 in range(0, gu.shape[0], 32768):
        n = min(32768, gu.shape[0] - t0)
        _check(library().ms_act_mul(gu[t0:].data_ptr(), out[t0:].data_ptr(), int(gu.dtype == BF16), n, inter, int(block), act, limit,
                                    _stream()), "act_mul")
    return out


def gated_linear(x: torch.Tensor, gate_up: torch.Tensor, activation: str = "silu", out_dtype=None, block: int = 0,
                 limit: float | None = None):
    """``act(x gate^T) * (x up^T)`` for ``gate_up [2 I, K]`` laid out as ``act_mul`` describes. With
    interleaved bfloat16 weights the activation runs in the matrix kernel's epilogue where a kernel
    for the shape exists (few rows: no partial sums leave the kernel; many rows: the gate/up matrix is
    never written); otherwise the product and the activation are two kernels."""
    act = _activation(activation, limit)
    _dev(x, "x", (F32, BF16), 2)
    _dev(gate_up, "gate_up", (F32, BF16), 2)
    m, k = x.shape
    if gate_up.shape[1] != k or gate_up.shape[0] % 2:
        raise ValueError(f"gated_linear: x is [{m}, {k}], gate_up is {tuple(gate_up.shape)}")
    inter = gate_up.shape[0] // 2
    if block == GATE_BLOCK and gate_up.dtype == BF16 and out_dtype == BF16 and m > 0 and activation not in ACTIVATIONS_WITH_LIMIT:
        xa = cast(x, BF16)
        out = torch.empty((m, inter), dtype=BF16, device=x.device)
        rc = library().ms_gemm_bf16_gated(xa.data_ptr(), gate_up.data_ptr(), out.data_ptr(), m, inter, k, k, act, _stream())
        if rc == 0:
            return out
        if rc != 2:  # 2: no fused kernel for this shape
            _check(rc, "gemm_bf16_gated")
    gu = linear(x, gate_up, out_dtype=out_dtype, defer=True)
    return act_mul(gu, activation, out_dtype=out_dtype, block=block, limit=limit)


def cast(x: torch.Tensor, dtype) -> torch.Tensor:
    if x.dtype == dtype:
        return x
    _dev(x, "x", (F32, BF16))
    if dtype not in (F32, BF16):
        raise TypeError(f"unsupported dtype {dtype}")
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    _check(library().ms_cast(x.data_ptr(), int(x.dtype == BF16), out.data_ptr(), int(dtype == BF16), x.numel(), _stream()),
           "cast")
    return out


# ------------------------------------------------------------------------------------- matrix products

SMALL_M = 64  # rows up to which the split-K weight-streaming kernel runs
MAX_STEP_TOKENS = 65535  # rows one launch of the matrix and elementwise kernels takes (a grid dimension)


def linear(x: torch.Tensor, weight: torch.Tensor, out_dtype=None, accumulate_into: torch.Tensor | None = None,
           defer: bool = False, out: torch.Tensor | None = None):
    """``x [M, K] @ weight [N, K]^T``. Either returns a new ``[M, N]`` tensor of ``out_dtype``, or adds
    the product into the float32 tensor ``accumulate_into`` (the residual stream) and returns None.
    The weight's dtype picks the arithmetic: float32 weights run the true 32-bit kernel (``x`` is
    widened first if needed), bfloat16 weights the matrix-core kernels with float32 accumulation.

    ``defer=True`` allows the result to come back as a ``SplitSum`` (partial sums that the consuming
    kernel adds up) where the small-M kernel produced it in that form; with ``accumulate_into`` the
    returned ``SplitSum`` is what still has to be added to that tensor.

    ``out``: a float32 ``[M, N]`` view of a wider matrix (unit column stride, rows a multiple of four floats apart and
    the first element 16-byte aligned) that receives the product; it is returned. Several products then share one
    matrix whose columns a later kernel reads side by side."""
    _dev(x, "x", (F32, BF16), 2)
    _dev(weight, "weight", (F32, BF16), 2)
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise ValueError(f"linear: x is [{m}, {k}], weight is {tuple(weight.shape)}")
    ldc = n
    if out is not None:
        if accumulate_into is not None or defer:
            raise ValueError("linear: out= goes with neither accumulate_into nor defer")
        if not (isinstance(out, torch.Tensor) and out.is_cuda and out.dtype == F32 and out.dim() == 2 and tuple(out.shape) == (m, n)
                and out.stride(1) == 1 and out.stride(0) >= n and out.stride(0) % 4 == 0 and out.data_ptr() % 16 == 0):
            raise ValueError(f"linear: out must be a float32 [{m}, {n}] view with unit column stride, rows a multiple of 4 floats "
                             "apart and a 16-byte aligned start")
        ldc = out.stride(0)
    if accumulate_into is not None:
        _dev(accumulate_into, "accumulate_into", F32, 2)
        if tuple(accumulate_into.shape) != (m, n):
            raise ValueError(f"linear: accumulator is {tuple(accumulate_into.shape)}, expected {(m, n)}")
    elif out is None and out_dtype not in (F32, BF16):
        raise TypeError(f"unsupported output dtype {out_dtype}")
    lib = library()
    if weight.dtype == BF16 and m <= SMALL_M:
        xa = cast(x, BF16)
        splits = lib.ms_gemm_bf16_small_splits(m, n, k)
        if splits == 1 and accumulate_into is None and out is None and out_dtype == F32:
            res = torch.empty((m, n), dtype=F32, device=x.device)  # the single partial sum is the result
            _check(lib.ms_gemm_bf16_small(xa.data_ptr(), weight.data_ptr(), res.data_ptr(), None, 1, 0, m, n, k, k, n,
                                          _stream()), "gemm_bf16_small")
            return res
        parts = torch.empty((splits, m, n), dtype=F32, device=x.device)
        if defer:
            _check(lib.ms_gemm_bf16_small(xa.data_ptr(), weight.data_ptr(), parts.data_ptr(), None, 1, 0, m, n, k, k, n,
                                          _stream()), "gemm_bf16_small")
            return SplitSum(parts)
        if out is not None:
            res = out
        else:
            res = accumulate_into if accumulate_into is not None else torch.empty((m, n), dtype=out_dtype, device=x.device)
        mode = 2 if accumulate_into is not None else (1 if res.dtype == F32 else 0)
        _check(lib.ms_gemm_bf16_small(xa.data_ptr(), weight.data_ptr(), parts.data_ptr(), res.data_ptr(), mode, 1, m, n, k,
                                      k, ldc, _stream()), "gemm_bf16_small")
        return None if accumulate_into is not None else res
    if weight.dtype == BF16 and defer:
        splits = lib.ms_gemm_bf16_tile_splits(m, n, k)
        if splits > 1:  # few output tiles: split K over the grid and leave the sum to the consumer
            xa = cast(x, BF16)
            parts = torch.empty((splits, m, n), dtype=F32, device=x.device)
            _check(lib.ms_gemm_bf16(xa.data_ptr(), weight.data_ptr(), parts.data_ptr(), 1, m, n, k, k, n, splits, _stream()),
                   "gemm_bf16")
            return SplitSum(parts)
    if out is not None:
        res = out
    else:
        res = accumulate_into if accumulate_into is not None else torch.empty((m, n), dtype=out_dtype, device=x.device)
    if weight.dtype == F32:
        xa = cast(x, F32)
        mode = 1 if accumulate_into is not None else (0 if res.dtype == F32 else 2)
        _check(lib.ms_gemm_f32(xa.data_ptr(), weight.data_ptr(), res.data_ptr(), mode, m, n, k, k, ldc, _stream()), "gemm_f32")
    else:
        xa = cast(x, BF16)
        mode = 2 if accumulate_into is not None else (1 if res.dtype == F32 else 0)
        _check(lib.ms_gemm_bf16(xa.data_ptr(), weight.data_ptr(), res.data_ptr(), mode, m, n, k, k, ldc, 1, _stream()), "gemm_bf16")
    return None if accumulate_into is not None else res


def tile_shape(m: int, n: int, k: int, splits: int = 1, gated: bool = False) -> tuple[int, int] | None:
    """``(rows, columns)`` of the tile that ``linear`` (or, with ``gated``, ``gated_linear`` with ``n = 2 I``)
    runs a bfloat16 product of more than ``SMALL_M`` contiguous rows with; None where the shape takes the
    kernel that stages its slabs through registers."""
    code = library().ms_gemm_bf16_tile_shape(m, n, k, k, splits, int(gated))
    return divmod(code, 1000) if code else None


def add_pending(residual: torch.Tensor, pending: SplitSum | None) -> None:
    """``residual += pending`` for callers whose next kernel cannot take a pending sum itself."""
    if pending is None:
        return
    _dev(residual, "residual", F32, 2)
    _check_split(pending, "pending", residual.shape)
    m, n = residual.shape
    _check(library().ms_splitk_reduce(pending.parts.data_ptr(), residual.data_ptr(), 2, pending.splits, m, n, n, _stream()),
           "splitk_reduce")


# ------------------------------------------------------------------------------------- mixture of experts

MOE_MAX_EXPERTS = 512  # MOE_MAX_EXPERTS in csrc/moe.hip
MOE_MAX_TOP = 64
MOE_SMALL_TILE_PAIRS = 16  # (token, expert) pairs per expert, on average, up to which a step runs 16-pair tiles
MOE_LARGE_TILE_PAIRS = 128  # ... and from which it runs 128-pair tiles (widths that are multiples of 64)


def moe_route(logits, bias: torch.Tensor | None, top: int, scoring: str = "chosen_softmax", groups: int = 1, keep: int = 1):
    """Per row of the float32 router logits ``[T, E]``: the ``top`` chosen outputs, best first (ties: the lower index), as
    int32 ``[T, top]``, and their weights, float32 ``[T, top]``. The logits may be a ``SplitSum``: the kernel adds the
    partial sums itself.

    ``scoring="chosen_softmax"``: the choice goes by ``logits + bias``, the weights are the softmax over the chosen values
    alone. ``scoring="softmax"``: ``s = softmax(logits)`` over all ``E`` outputs; the choice goes by ``s + bias`` (a
    correction that only the choice sees), the weights are the chosen outputs' ``s`` as they stand; with ``groups > 1``
    the outputs form that many equal groups of neighbours, a group's score is the largest ``s + bias`` in it, and only
    outputs of the ``keep`` best groups can be chosen."""
    if isinstance(logits, SplitSum):
        parts, splits, stride = logits.parts, logits.splits, logits.stride
        _dev(parts, "logits", F32, 3)
        t, e = logits.shape
    else:
        _dev(logits, "logits", F32, 2)
        parts, splits, stride = logits, 1, 0
        t, e = logits.shape
    if not 1 <= top <= e:
        raise ValueError(f"top {top} of {e} experts")
    if e > MOE_MAX_EXPERTS or top > MOE_MAX_TOP:
        raise ValueError(f"{e} experts / top {top}: the routing kernel takes up to {MOE_MAX_EXPERTS} experts and {MOE_MAX_TOP} choices")
    if scoring not in ("chosen_softmax", "softmax"):
        raise NotImplementedError(f"router scoring {scoring!r}: 'chosen_softmax' or 'softmax'")
    if bias is not None:
        _dev(bias, "bias", (F32, BF16), 1)
        if bias.shape[0] != e:
            raise ValueError(f"the router's bias has {bias.shape[0]} elements for {e} experts")
    ids = torch.empty((t, top), dtype=I32, device=parts.device)
    weights = torch.empty((t, top), dtype=F32, device=parts.device)
    if scoring == "softmax":
        if groups < 1 or e % groups or not 1 <= keep <= groups:
            raise ValueError(f"{e} router outputs in {groups} groups of which {keep} are kept")
        if top > (e // groups) * keep:
            raise ValueError(f"top {top} of the {(e // groups) * keep} outputs in the kept groups")
        _check(library().ms_moe_route_scored(parts.data_ptr(), e, splits, stride, _ptr(bias), int(bias is not None and bias.dtype == BF16),
                                             t, e, top, int(groups), int(keep), ids.data_ptr(), weights.data_ptr(), _stream()),
               "moe_route_scored")
        return ids, weights
    if groups != 1:
        raise NotImplementedError("groups of experts go with scoring='softmax'")
    _check(library().ms_moe_route(parts.data_ptr(), e, splits, stride, _ptr(bias), int(bias is not None and bias.dtype == BF16), t, e,
                                  top, ids.data_ptr(), weights.data_ptr(), _stream()), "moe_route")
    return ids, weights


def moe_experts(x: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, gate: torch.Tensor | None, up: torch.Tensor,
                down: torch.Tensor, activation: str, stream: torch.Tensor) -> None:
    """``stream[t] += sum_j weights[t, j] * expert_e(x[t])`` with ``e = ids[t, j]``, the sum in ascending ``j``. A gated
    expert is ``down[e] (act(gate[e] x) * (up[e] x))``; with ``gate=None`` it is ``down[e] act(up[e] x)``. An id of
    ``E`` (the number of experts that have weights) or more names an identity expert: its term is ``weights[t, j] * x[t]``.
    ``x [T, W]`` in the compute dtype, ``gate`` / ``up`` ``[E, F, W]`` and ``down [E, W, F]`` in the same, ``stream`` float32
    ``[T, W]``. The step's (token, expert) pairs are sorted by expert on the device and every expert's run is multiplied
    in tiles (bfloat16: on the matrix cores; float32: fused multiply-adds in ascending k); the launches cover the most
    tiles the step can have, so nothing is read back and a captured step replays."""
    gated = gate is not None
    act = _activation(activation, gated=gated)
    if act == ACTIVATIONS["swiglu_clamped"]:
        raise NotImplementedError(f"activation {activation!r} is not of the form act(gate) * up")
    _dev(x, "x", (F32, BF16), 2)
    for w, nm in ((gate, "gate"), (up, "up"), (down, "down")):
        if w is not None:
            _dev(w, nm, x.dtype, 3)
    _dev(ids, "ids", I32, 2)
    _dev(weights, "weights", F32, 2)
    _dev(stream, "stream", F32, 2)
    t, width = x.shape
    e, f = up.shape[0], up.shape[1]
    top = ids.shape[1]
    if (gated and gate.shape != (e, f, width)) or up.shape != (e, f, width) or down.shape != (e, width, f):
        raise ValueError(f"expert weights {tuple(up.shape)} / {tuple(down.shape)} do not fit x {tuple(x.shape)}")
    if ids.shape[0] != t or tuple(weights.shape) != tuple(ids.shape) or tuple(stream.shape) != (t, width):
        raise ValueError("ids, weights and stream must have one row per row of x")
    if e > MOE_MAX_EXPERTS:
        raise ValueError(f"{e} experts: the kernels take up to {MOE_MAX_EXPERTS}")
    if t == 0:
        return
    if t > MAX_STEP_TOKENS:
        raise ValueError(f"{t} rows: one launch takes at most {MAX_STEP_TOKENS}")
    pairs = t * top
    bf = x.dtype == BF16
    tile_rows = 16 if bf and pairs <= MOE_SMALL_TILE_PAIRS * e else 64
    if bf and pairs >= MOE_LARGE_TILE_PAIRS * e and width % 64 == 0 and f % 64 == 0 and not any(
            w.data_ptr() % 16 for w in (x, gate, up, down) if w is not None):
        tile_rows = 128  # both products then run tiles of 128 pairs staged through LDS
    max_tiles = -(-pairs // tile_rows) + min(e, pairs)
    dev = x.device
    order = torch.empty((pairs,), dtype=I32, device=dev)
    tiles = torch.empty((3, max_tiles), dtype=I32, device=dev)
    lib = library()
    _check(lib.ms_moe_plan(ids.data_ptr(), pairs, e, tile_rows, max_tiles, order.data_ptr(), tiles[0].data_ptr(), tiles[1].data_ptr(),
                           tiles[2].data_ptr(), _stream()), "moe_plan")
    plan = (order.data_ptr(), tiles[0].data_ptr(), tiles[1].data_ptr(), tiles[2].data_ptr())
    h = torch.empty((pairs, f), dtype=x.dtype, device=dev)
    _check(lib.ms_moe_gemm(x.data_ptr(), width, (gate if gated else up).data_ptr(), up.data_ptr() if gated else None, h.data_ptr(), int(bf),
                           1 if gated else 2, *plan, None, max_tiles, top, f, width, tile_rows, act, _stream()), "moe_gemm")
    y = torch.empty((pairs, width), dtype=F32, device=dev)
    _check(lib.ms_moe_gemm(h.data_ptr(), f, down.data_ptr(), None, y.data_ptr(), int(bf), 0, *plan, weights.data_ptr(), max_tiles, top,
                           width, f, tile_rows, act, _stream()), "moe_gemm")
    _check(lib.ms_moe_combine(stream.data_ptr(), y.data_ptr(), t, top, width, ids.data_ptr(), weights.data_ptr(), x.data_ptr(), int(bf),
                              width, e, _stream()), "moe_combine")


# ------------------------------------------------------------------------------------- attention


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, magnitude: float = 1.0) -> torch.Tensor:
    """Cosines and sines of the rotation angles ``float32(position) * inv_freq[j]`` of a step's tokens, each multiplied
    by ``magnitude``: float32 ``[T, 2 * len(inv_freq)]``, a row holding the cosines, then the sines. Made once per step
    and shared by all layers that rotate by the same frequencies."""
    _dev(positions, "positions", I32, 1)
    _dev(inv_freq, "inv_freq", F32, 1)
    t, half = positions.shape[0], inv_freq.shape[0]
    out = torch.empty((t, 2 * half), dtype=F32, device=positions.device)
    _check(library().ms_rope_table(positions.data_ptr(), inv_freq.data_ptr(), out.data_ptr(), t, half, float(magnitude), _stream()),
           "rope_table")
    return out


# Which elements of a head make pair j of a rotation, and the numbers the kernels know the pairings by (MS_ROPE_* in
# csrc/common.h): "halves" (j, j + dim/2), "adjacent" (2j, 2j + 1).
ROTATION_PAIRINGS = {"halves": 0, "adjacent": 1}


def _pairing(name: str) -> int:
    try:
        return ROTATION_PAIRINGS[name]
    except KeyError:
        raise NotImplementedError(f"rotation pairing {name!r}: the kernels know {sorted(ROTATION_PAIRINGS)}") from None


def qk_norm_rope_store(qkv, slots, q_weight, k_weight, eps, rope, k_cache, v_cache,
                       num_heads, num_kv_heads, head_dim, out_dtype=None, pairing: str = "halves") -> torch.Tensor:
    """From ``qkv [T, (Hq + 2 Hkv) D]`` (a tensor, or a ``SplitSum`` of it): per-head RMSNorm of q and k
    (if weights are given), rotation of the first ``rope.shape[1]`` elements of each head, in pairs as
    ``pairing`` names them, by the angles
    of ``rope`` (a ``rope_table`` of these tokens; None: no rotation), k and v stored into the cache
    pages at ``slots`` (skipped when ``slots`` is None). Returns the tensor that holds the finished
    queries in its first ``Hq * D`` columns: ``qkv`` itself (written in place), or for a ``SplitSum`` a
    new ``[T, Hq D]`` tensor of ``out_dtype``."""
    width = (num_heads + 2 * num_kv_heads) * head_dim
    if isinstance(qkv, SplitSum):
        _dev(qkv.parts, "qkv", F32, 3)
        t = qkv.shape[0]
        if qkv.shape[1] != width or out_dtype not in (F32, BF16):
            raise ValueError(f"qkv partial sums have width {qkv.shape[1]}, expected {width}, and need an output dtype")
        dtype = out_dtype
        q_out = torch.empty((t, num_heads * head_dim), dtype=dtype, device=qkv.parts.device)
        src, parts, splits, stride = None, qkv.parts.data_ptr(), qkv.splits, qkv.stride
    else:
        _dev(qkv, "qkv", (F32, BF16), 2)
        t = qkv.shape[0]
        if qkv.shape[1] != width:
            raise ValueError(f"qkv has width {qkv.shape[1]}, expected {width}")
        dtype = qkv.dtype
        q_out = qkv
        src, parts, splits, stride = qkv.data_ptr(), None, 0, 0
    if head_dim > 256 or head_dim < 1:
        raise ValueError(f"head_dim {head_dim} is outside the kernels' range 1..256")
    w_bf16 = 0
    if q_weight is not None:
        for w, nm in ((q_weight, "q_norm"), (k_weight, "k_norm")):
            _dev(w, nm, (F32, BF16), 1)
            if w.shape[0] != head_dim:
                raise ValueError(f"{nm} weight has {w.shape[0]} elements for head_dim {head_dim}")
        if q_weight.dtype != k_weight.dtype:
            raise TypeError("q_norm and k_norm weights differ in dtype")
        w_bf16 = int(q_weight.dtype == BF16)
    page_size = 1
    if slots is not None:
        _dev(slots, "slots", I32, 1)
        if slots.shape[0] != t:
            raise ValueError("one slot per token is needed")
        page_size = _check_caches(k_cache, v_cache, dtype, num_kv_heads, head_dim)
    rot_dim, pair = 0, _pairing(pairing)
    if rope is not None:
        _dev(rope, "rope", F32, 2)
        rot_dim = rope.shape[1]
        if rope.shape[0] != t or rot_dim % 2 or rot_dim > head_dim or rot_dim < 2:
            raise ValueError(f"rotation table is {tuple(rope.shape)}; {t} tokens and an even width up to {head_dim} are needed")
    _check(library().ms_qk_norm_rope_store(
        src, parts, splits, stride, q_out.data_ptr(), q_out.shape[1], int(dtype == BF16), _ptr(slots),
        _ptr(q_weight), _ptr(k_weight), w_bf16, float(eps), _ptr(rope), int(rot_dim), pair,
        _ptr(k_cache) if slots is not None else None, _ptr(v_cache) if slots is not None else None, t, num_heads,
        num_kv_heads, head_dim, page_size, _stream()), "qk_norm_rope_store")
    return q_out


def _check_caches(k_cache, v_cache, dtype, num_kv_heads, head_dim, value_dim: int | None = None) -> int:
    """Keys ``[pages, Hkv, page, D]``, values ``[pages, Hkv, Dv, page]`` (``Dv = D`` unless ``value_dim`` is
    given); returns the page size."""
    _dev(k_cache, "k_cache", dtype, 4)
    _dev(v_cache, "v_cache", dtype, 4)
    page = k_cache.shape[2]
    dv = head_dim if value_dim is None else value_dim
    if tuple(k_cache.shape[1:]) != (num_kv_heads, page, head_dim):
        raise ValueError(f"k_cache is {tuple(k_cache.shape)}, expected [pages, {num_kv_heads}, page, {head_dim}]")
    if tuple(v_cache.shape) != (k_cache.shape[0], num_kv_heads, dv, page):
        raise ValueError(f"v_cache is {tuple(v_cache.shape)}, expected [{k_cache.shape[0]}, {num_kv_heads}, {dv}, {page}]")
    return page


TILED_ROWS = 64  # query rows (tokens x the heads of a group) a block of the tiled attention kernels owns
MFMA_SPLIT_BLOCKS = 256  # blocks a step of single tokens aims for when it shares a token's keys among blocks
MFMA_DECODE_GROUP = 8  # query heads per key head from which single-token rows run the tiled matrix-core kernel too
GENERIC_MAX_HEAD_DIM = 1024  # head sizes the generic attention kernel takes (MAX_WIDE_HEAD_DIM in csrc/attention.hip)


def _check_special_caches(k_cache, v_cache, dtype, num_kv_heads, head_dim, value_dim, value_share, values_in_keys) -> int:
    """Keys ``[pages, Hkv, page, D]``; values ``[pages, Hkv / value_share, Dv, page]``, or none where the keys' rows
    hold them. Returns the page size."""
    _dev(k_cache, "k_cache", dtype, 4)
    page = k_cache.shape[2]
    if tuple(k_cache.shape[1:]) != (num_kv_heads, page, head_dim):
        raise ValueError(f"k_cache is {tuple(k_cache.shape)}, expected [pages, {num_kv_heads}, page, {head_dim}]")
    if value_share < 1 or num_kv_heads % value_share:
        raise ValueError(f"{num_kv_heads} key heads cannot share values in runs of {value_share}")
    if values_in_keys:
        if v_cache is not None or value_share != 1 or value_dim > head_dim:
            raise ValueError("values inside the keys: no value cache, no sharing, and a value size up to the key size")
        return page
    _dev(v_cache, "v_cache", dtype, 4)
    want = (k_cache.shape[0], num_kv_heads // value_share, value_dim, page)
    if tuple(v_cache.shape) != want:
        raise ValueError(f"v_cache is {tuple(v_cache.shape)}, expected {list(want)}")
    return page


PREFILL_BIG_BLOCKS = 640  # from this many 128-row blocks on, the prefill attention runs 128-row blocks
DECODE_TARGET_BLOCKS = 512  # workgroups the split decode kernel aims for
DECODE_MIN_CHUNKS = 4  # 32-token chunks a split should at least hold


def decode_splits(rows: int, num_kv_heads: int, max_kv_len: int) -> int:
    """How many ways the keys of each sequence are split in the decode kernel: enough workgroups to
    fill the chip, but no split shorter than a few chunks."""
    by_fill = -(-DECODE_TARGET_BLOCKS // max(1, rows * num_kv_heads))
    by_len = max(1, -(-max_kv_len // 32) // DECODE_MIN_CHUNKS)
    return max(1, min(by_fill, by_len))


def decode_attention_fusable(qkv, batch, q_weight, k_weight, rope, k_cache, v_cache, num_heads, num_kv_heads, head_dim,
                             pairing: str = "halves") -> bool:
    """Whether ``decode_attention_fused`` takes this step: every row brings one token, the qkv
    projection comes as partial sums, bfloat16 cache with 16-token pages, a head size of 64 or 128, at
    most 16 query heads per KV head, bfloat16 norm weights (or none), rotation over the whole head in
    pairs (j, j + D/2) (or none)."""
    return (isinstance(qkv, SplitSum) and (rope is None or pairing == "halves") and batch.is_decode and batch.decode_tokens is None
            and k_cache.dtype == BF16 and v_cache.dtype == BF16 and k_cache.dim() == 4 and k_cache.shape[2] == 16
            and head_dim in (64, 128) and num_heads % num_kv_heads == 0 and num_heads // num_kv_heads <= 16
            and qkv.stride % 4 == 0
            and (q_weight is None) == (k_weight is None) and (q_weight is None or (q_weight.dtype == BF16 and k_weight.dtype == BF16))
            and (rope is None or rope.shape[1] == head_dim))


MERGE_PROJECT_MAX_ROWS = 16  # rows up to which the splits' reduction and the output projection are one kernel
MERGE_PROJECT_MAX_SPLITS = 64


def decode_attention_fused(qkv, q_weight, k_weight, eps, rope, store, k_cache, v_cache, block_table, batch,
                           num_heads, num_kv_heads, head_dim, scale, window, project: torch.Tensor | None = None):
    """``qk_norm_rope_store`` and ``paged_attention`` of a step of single tokens in one kernel, from the
    partial sums ``qkv`` (a ``SplitSum`` of ``[T, (Hq + 2 Hkv) D]``): the queries never go to memory,
    and with ``store`` the new token's key and value are written to the cache by the block that uses
    them first. Returns bfloat16 ``[T, Hq * D]``. ``decode_attention_fusable`` says when this applies.

    ``project``: the output projection's weight ``[N, Hq * D]`` (bfloat16). Where the keys were split
    (they are whenever the step has few rows) and the step has up to ``MERGE_PROJECT_MAX_ROWS`` rows,
    the reduction of the splits and that projection run as one kernel and a ``SplitSum`` of
    ``[T, N]`` is returned instead of the attention's output: no reduction kernel, and the attention's
    output never goes to memory."""
    if not decode_attention_fusable(qkv, batch, q_weight, k_weight, rope, k_cache, v_cache, num_heads, num_kv_heads, head_dim):
        raise ValueError("this step cannot run the fused decode attention")
    _dev(qkv.parts, "qkv", F32, 3)
    t = qkv.shape[0]
    if qkv.shape[1] != (num_heads + 2 * num_kv_heads) * head_dim:
        raise ValueError(f"qkv partial sums have width {qkv.shape[1]}, expected {(num_heads + 2 * num_kv_heads) * head_dim}")
    page = _check_caches(k_cache, v_cache, BF16, num_kv_heads, head_dim)
    if not scale > 0:
        raise ValueError(f"the attention scale must be positive, not {scale}")
    if q_weight is not None:
        for w, nm in ((q_weight, "q_norm"), (k_weight, "k_norm")):
            _dev(w, nm, BF16, 1)
            if w.shape[0] != head_dim:
                raise ValueError(f"{nm} weight has {w.shape[0]} elements for head_dim {head_dim}")
    if rope is not None:
        _dev(rope, "rope", F32, 2)
        if rope.shape[0] != t:
            raise ValueError("one row of the rotation table per token is needed")
    _dev(block_table, "block_table", I32, 2)
    _dev(batch.token_row, "token_row", I32, 1)
    _dev(batch.positions, "positions", I32, 1)
    if batch.token_row.shape[0] != t or batch.positions.shape[0] != t or block_table.shape[0] < batch.num_rows:
        raise ValueError("batch metadata does not match the number of tokens or rows")
    dev = qkv.parts.device
    lib = library()
    splits = decode_splits(t, num_kv_heads, batch.max_kv_len)
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty((t * num_heads * splits * head_dim,), dtype=F32, device=dev)
        part_ml = torch.empty((t * num_heads * splits * 2,), dtype=F32, device=dev)
    merged = None  # partial sums of the projection, where one kernel reduces the splits and projects
    if (project is not None and MERGE_PROJECT_MAX_ROWS > 0 and 1 < splits <= MERGE_PROJECT_MAX_SPLITS
            and t <= MERGE_PROJECT_MAX_ROWS):
        _dev(project, "project", BF16, 2)
        n = project.shape[0]
        out_splits = lib.ms_attention_merge_project_splits(t, num_heads, head_dim, splits, n)
        if project.shape[1] == num_heads * head_dim and out_splits >= 1:
            merged = torch.empty((out_splits, t, n), dtype=F32, device=dev)
    out = None if merged is not None else torch.empty((t, num_heads * head_dim), dtype=BF16, device=dev)
    _check(lib.ms_attention_decode_fused_bf16(
        qkv.parts.data_ptr(), qkv.splits, qkv.stride, _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(rope),
        ROTATION_PAIRINGS["halves"], int(bool(store)),
        k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), block_table.shape[1], None,
        batch.token_row.data_ptr(), batch.positions.data_ptr(), _ptr(out), _ptr(part_o), _ptr(part_ml), t, splits,
        num_heads, num_kv_heads, head_dim, page, float(scale), int(window), int(merged is None), _stream()),
        "attention_decode_fused")
    if merged is None:
        return out
    _check(lib.ms_attention_merge_project(part_o.data_ptr(), part_ml.data_ptr(), project.data_ptr(), merged.data_ptr(), t,
                                          num_heads, head_dim, splits, merged.shape[2], _stream()), "attention_merge_project")
    return SplitSum(merged)


def paged_attention(qkv, k_cache, v_cache, block_table, batch, num_heads, num_kv_heads, head_dim, scale, window,
                    value_dim: int | None = None, keep_first: int = 0, exact_weights: bool = False, softcap: float = 0.0,
                    sinks: torch.Tensor | None = None, value_share: int = 1, values_in_keys: bool = False,
                    out_dtype=None):
    """Attention of the batch's new tokens over the cache. ``qkv [T, >= Hq D]`` holds the queries
    in its first ``Hq * D`` columns. Returns ``[T, Hq * Dv]`` (``Dv = D`` unless ``value_dim`` is given).
    A query at position p sees keys ``max(0, p - window + 1) .. p`` (``window == 0``: all up to p) and, with a
    window, the keys ``0 .. keep_first - 1`` as well.

    bfloat16 with 16-token pages and a head size of 64 or 128: rows that bring one token run the
    split decode kernel, rows that bring several the tiled prefill kernel. Everything else (float32,
    other head sizes or page sizes, values of another size than the keys, kept first keys, or
    ``exact_weights``: softmax weights that must meet the values unrounded) runs the generic kernel.

    Options of the generic kernel (float32 arithmetic throughout, head sizes up to 1024) and of the second tiled
    matrix-core kernel (bfloat16 storage, 16-token pages, key sizes that are multiples of 32 and value sizes that are
    multiples of 16, up to 64 query heads per key head; softmax weights unrounded; rows of several tokens, and steps of
    single tokens only, whose keys are shared among a block's waves and among blocks):
    ``softcap > 0`` bounds a scaled score ``s`` to ``softcap * tanh(s / softcap)``; ``sinks`` (float32 ``[Hq]``) adds
    ``exp(sinks[h])`` to head ``h``'s softmax denominator; ``value_share = n`` lets ``n`` consecutive key heads weigh
    the same value head (``v_cache`` then has ``Hkv / n`` heads); ``values_in_keys`` takes the first ``Dv`` elements
    of each key row as that token's value (``v_cache`` is None); ``out_dtype=torch.float32`` returns the result
    unrounded whatever the cache's dtype."""
    _dev(qkv, "qkv", (F32, BF16), 2)
    t = qkv.shape[0]
    dv = head_dim if value_dim is None else int(value_dim)
    out_f32 = out_dtype == F32 and qkv.dtype != F32
    if out_dtype not in (None, F32, qkv.dtype):
        raise TypeError(f"the result comes in the queries' dtype or in float32, not {out_dtype}")
    special = bool(softcap) or sinks is not None or value_share != 1 or values_in_keys or out_f32
    if special:
        page = _check_special_caches(k_cache, v_cache, qkv.dtype, num_kv_heads, head_dim, dv, value_share, values_in_keys)
        if sinks is not None:
            _dev(sinks, "sinks", F32, 1)
            if sinks.shape[0] != num_heads:
                raise ValueError(f"{sinks.shape[0]} sinks for {num_heads} query heads")
        if not softcap >= 0:
            raise ValueError(f"softcap must not be negative, got {softcap}")
    else:
        page = _check_caches(k_cache, v_cache, qkv.dtype, num_kv_heads, head_dim, dv)
    limit = GENERIC_MAX_HEAD_DIM if special else 256
    if not (1 <= head_dim <= limit and 1 <= dv <= limit):
        raise ValueError(f"head sizes {head_dim} / {dv} are not supported: the attention kernels take sizes up to {limit}")
    if keep_first < 0 or window < 0:
        raise ValueError("window and keep_first must not be negative")
    if num_heads % num_kv_heads:
        raise ValueError(f"{num_heads} query heads are no multiple of {num_kv_heads} KV heads")
    if qkv.shape[1] < num_heads * head_dim:
        raise ValueError("qkv is narrower than the query heads")
    if not scale > 0:
        raise ValueError(f"the attention scale must be positive, not {scale}")  # the kernels scale masked scores too
    _dev(block_table, "block_table", I32, 2)
    _dev(batch.token_row, "token_row", I32, 1)
    _dev(batch.positions, "positions", I32, 1)
    if batch.token_row.shape[0] != t or batch.positions.shape[0] != t or block_table.shape[0] < batch.num_rows:
        raise ValueError("batch metadata does not match the number of tokens or rows")
    out = torch.empty((t, num_heads * dv), dtype=F32 if out_f32 else qkv.dtype, device=qkv.device)
    lib = library()
    common = (block_table.data_ptr(), block_table.shape[1])
    meta = (batch.token_row.data_ptr(), batch.positions.data_ptr(), out.data_ptr())
    n_dec = batch.num_decode_tokens
    fast = (qkv.dtype == BF16 and page == 16 and head_dim in (64, 128) and num_heads // num_kv_heads <= 16
            and qkv.shape[1] % 8 == 0 and dv == head_dim and not (window and keep_first) and not exact_weights and not special)
    if not fast:
        generic = (qkv.data_ptr(), qkv.shape[1], k_cache.data_ptr(), _ptr(v_cache), int(qkv.dtype == BF16), *common)
        shape = (num_heads, num_kv_heads, head_dim, dv, page, float(scale), int(window), int(keep_first))
        extra = (float(softcap), _ptr(sinks), int(value_share), int(values_in_keys), int(out_f32))
        tile_tokens = 0 if special else lib.ms_paged_attention_tiled_tokens(num_heads // num_kv_heads, head_dim, dv)
        lens = getattr(batch, "row_lens", None)
        group = num_heads // num_kv_heads
        wide = (special and lens is not None and qkv.dtype == BF16 and qkv.shape[1] % 8 == 0 and not values_in_keys
                and lib.ms_paged_attention_tiled_mfma_wide_chunk(group, head_dim, dv, page, 1))
        # On the matrix cores: rows that bring several tokens; single-token rows too where a key head serves so many query
        # heads that they fill a wave's 16 rows, or where the step has no other rows (its tokens' keys are then shared
        # among waves and blocks, which pays whatever the group's size).
        single_too = wide and (group >= MFMA_DECODE_GROUP or n_dec == t)
        wide_rows = t if single_too else (t - n_dec if wide else 0)
        if wide_rows:
            all_rows = wide_rows == t
            if not all_rows and n_dec:
                _check(lib.ms_paged_attention_generic(*generic, _ptr(batch.decode_tokens), *meta, n_dec, *shape, DECODE_GENERIC_WAVES,
                                                      *extra, _stream()), "paged_attention")
            first, count, tiles = _tiles_of_rows(batch, TILED_ROWS // group, qkv.device, all_rows)
            splits, part_o, part_ml = 0, None, None
            if all_rows and n_dec == t:
                # a step of single tokens: a block's four waves share a token's key tiles, and so many blocks share them
                # that the chip is full, each with at least a tile per wave
                heads16 = num_kv_heads * -(-group // 16)  # a block owns up to 16 of a key head's query heads
                runs = dv // wide  # the run of values a block owns in a step of single tokens
                key_tiles = -(-(min(batch.max_kv_len, window) if window else batch.max_kv_len) // 64) + 1
                splits = max(1, min(key_tiles // 4, -(-MFMA_SPLIT_BLOCKS // (t * heads16 * runs))))
                if splits > 1:
                    part_o = torch.empty((t * heads16 * runs * splits * 16 * wide,), dtype=F32, device=qkv.device)
                    part_ml = torch.empty((t * heads16 * runs * splits * 16 * 2,), dtype=F32, device=qkv.device)
            if block_table.shape[1] % 4:  # the kernel reads the four page ids of a key tile at once
                padded = torch.zeros((block_table.shape[0], -(-block_table.shape[1] // 4) * 4), dtype=I32, device=block_table.device)
                padded[:, : block_table.shape[1]] = block_table
                common = (padded.data_ptr(), padded.shape[1])
            _check(lib.ms_paged_attention_tiled_mfma_wide(
                qkv.data_ptr(), qkv.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), *common, first.data_ptr(), count.data_ptr(), tiles,
                batch.token_row.data_ptr(), batch.positions.data_ptr(), out.data_ptr(), int(out_f32), num_heads, num_kv_heads, head_dim,
                dv, page, float(scale), int(window), int(keep_first), float(softcap), _ptr(sinks), int(value_share), splits,
                _ptr(part_o), _ptr(part_ml), _stream()), "paged_attention_tiled_mfma_wide")
            return out
        if special and lens is not None and 0 < n_dec < t:
            # single-token rows walk their keys with several waves, the others with one wave per token and head
            _check(lib.ms_paged_attention_generic(*generic, _ptr(batch.decode_tokens), *meta, n_dec, *shape, DECODE_GENERIC_WAVES,
                                                  *extra, _stream()), "paged_attention")
            _check(lib.ms_paged_attention_generic(*generic, _ptr(batch.prefill_tokens), *meta, t - n_dec, *shape, 1, *extra,
                                                  _stream()), "paged_attention")
            return out
        if special and lens is not None and n_dec == t:
            _check(lib.ms_paged_attention_generic(*generic, None, *meta, t, *shape, DECODE_GENERIC_WAVES, *extra, _stream()),
                   "paged_attention")
            return out
        if not (exact_weights or keep_first or dv != head_dim) or not tile_tokens or lens is None:
            # the form whose sums have one order whatever the step looks like: float32 results stay bitwise equal
            _check(lib.ms_paged_attention_generic(*generic, None, *meta, t, *shape, 1, *extra, _stream()), "paged_attention")
            return out
        # rows that bring one token: several waves share a head's keys; rows that bring several: tiles of tokens in LDS
        if n_dec:
            _check(lib.ms_paged_attention_generic(*generic, _ptr(batch.decode_tokens), *meta, n_dec, *shape, DECODE_GENERIC_WAVES,
                                                  *extra, _stream()), "paged_attention")
        if n_dec < t:
            first, count, tiles = _tiles_of(batch, tile_tokens, qkv.device)
            if qkv.dtype == BF16 and qkv.shape[1] % 8 == 0 and lib.ms_paged_attention_tiled_mfma_ok(head_dim, dv, page):
                # on the matrix cores, with every float32 softmax weight cut into three bfloat16 pieces: nothing is rounded
                if block_table.shape[1] % 4:  # the kernel reads the four page ids of a key tile at once
                    wide = torch.zeros((block_table.shape[0], -(-block_table.shape[1] // 4) * 4), dtype=I32, device=block_table.device)
                    wide[:, : block_table.shape[1]] = block_table
                    common = (wide.data_ptr(), wide.shape[1])
                _check(lib.ms_paged_attention_tiled_mfma(qkv.data_ptr(), qkv.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), *common,
                                                         first.data_ptr(), count.data_ptr(), tiles, *meta, *shape, _stream()),
                       "paged_attention_tiled_mfma")
            else:
                _check(lib.ms_paged_attention_tiled(*generic, first.data_ptr(), count.data_ptr(), tiles, *meta, *shape, _stream()),
                       "paged_attention_tiled")
        return out
    if n_dec:
        splits = decode_splits(n_dec, num_kv_heads, batch.max_kv_len)
        part_o = part_ml = None
        if splits > 1:
            part_o = torch.empty((n_dec * num_heads * splits * head_dim,), dtype=F32, device=qkv.device)
            part_ml = torch.empty((n_dec * num_heads * splits * 2,), dtype=F32, device=qkv.device)
        _check(lib.ms_attention_decode_bf16(
            qkv.data_ptr(), qkv.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), *common, _ptr(batch.decode_tokens), *meta,
            _ptr(part_o), _ptr(part_ml), n_dec, splits, num_heads, num_kv_heads, head_dim, page, float(scale), int(window),
            _stream()), "attention_decode")
    if n_dec < t:
        if block_table.shape[1] % 4:  # the prefill kernel reads four page ids at once
            wide = torch.zeros((block_table.shape[0], -(-block_table.shape[1] // 4) * 4), dtype=I32, device=block_table.device)
            wide[:, : block_table.shape[1]] = block_table
            block_table = wide
            common = (block_table.data_ptr(), block_table.shape[1])
        group = num_heads // num_kv_heads
        # 128 query rows per block read K and V least often; 64 (each wave takes half of every key tile)
        # give short chains and more blocks. The latter until 128-row blocks alone fill the chip twice over.
        n_prefill = t - n_dec
        rows = 128 if (group > 64 or -(-n_prefill // (128 // group)) * num_kv_heads >= PREFILL_BIG_BLOCKS) else 64
        tile_tokens = lib.ms_attention_prefill_tile_tokens(group, rows)
        plan = _prefill_parts_plan(batch, tile_tokens, num_kv_heads, rows * head_dim * 4) if window == 0 else None
        if plan is not None:
            part_o = torch.empty((plan.slots * num_kv_heads * rows * head_dim,), dtype=F32, device=qkv.device)
            part_ml = torch.empty((plan.slots * num_kv_heads * rows * 2,), dtype=F32, device=qkv.device)
            _check(lib.ms_attention_prefill_parts_bf16(
                qkv.data_ptr(), qkv.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), *common, plan.table.data_ptr(),
                plan.entries, plan.merges, part_o.data_ptr(), part_ml.data_ptr(), rows, *meta, num_heads, num_kv_heads,
                head_dim, page, float(scale), _stream()), "attention_prefill_parts")
            return out
        first, count, tiles = batch.prefill_tiles(tile_tokens)
        _check(lib.ms_attention_prefill_bf16(
            qkv.data_ptr(), qkv.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), *common, first.data_ptr(), count.data_ptr(),
            tiles, rows, *meta, num_heads, num_kv_heads, head_dim, page, float(scale), int(window), _stream()),
            "attention_prefill")
    return out


def _tiles_of(batch, tile_tokens: int, device):
    """``build_prefill_tiles`` of a step, made once per tile size (the step's batch keeps them where it can)."""
    if hasattr(batch, "prefill_tiles"):
        return batch.prefill_tiles(tile_tokens)
    return build_prefill_tiles(batch.row_lens, batch.row_starts_host, tile_tokens, device)


def _tiles_of_rows(batch, tile_tokens: int, device, all_rows: bool):
    """Tiles of the rows that bring several tokens, or, ``all_rows``, of every row (a single token is a tile of one).
    A step of single tokens only gets its tiles from the device alone (one per token, in order), so that a captured
    graph can replay them."""
    if not all_rows:
        return _tiles_of(batch, tile_tokens, device)
    if batch.num_decode_tokens == batch.num_tokens:
        key = ("single-token tiles",)
        if key not in batch.memo:
            n = batch.num_tokens
            batch.memo[key] = (torch.arange(n, dtype=I32, device=device), torch.ones(n, dtype=I32, device=device), n)
        return batch.memo[key]
    key = ("tiles of all rows", tile_tokens)
    if key not in batch.memo:
        batch.memo[key] = build_prefill_tiles(batch.row_lens, batch.row_starts_host, tile_tokens, device, least=1)
    return batch.memo[key]


def build_prefill_tiles(row_lens, row_starts, tile_tokens: int, device, least: int = 2):
    """Tiles of at most ``tile_tokens`` consecutive new tokens of the rows that bring several tokens (at least
    ``least``): ``(first flat token index [n], token count [n], n)`` on the device, the tile deepest into its
    sequence (the most keys to visit) first."""
    tiles = []
    t = 0
    for n, s in zip(row_lens, row_starts):
        if n >= least:
            for a in range(0, n, tile_tokens):
                tiles.append((s + min(n, a + tile_tokens), t + a, min(tile_tokens, n - a)))
        t += n
    tiles.sort(key=lambda x: -x[0])
    host = torch.tensor([[f for _, f, _ in tiles], [c for _, _, c in tiles]], dtype=I32)
    dev = host.to(device, non_blocking=True)
    return dev[0], dev[1], len(tiles)


PREFILL_KEY_TILE = 64        # keys per iteration of the prefill attention kernel
PREFILL_RESIDENT_BLOCKS = 512  # blocks of it the chip holds at once (two per CU)
PREFILL_MIN_PART = 4         # key tiles: no part is made shorter than this
PREFILL_PARTS_LAUNCH_US = 8.0  # what the merge kernel costs beside the bytes it moves
PREFILL_PARTS_MARGIN = 1.5   # parts are made where they save this many times what they cost


class PrefillPartsPlan:
    """Tiles of new tokens whose keys are handed out in parts. ``table``: int32 on the device, per entry
    first token, token count, first key tile, end key tile, slot (-1: a whole tile), heaviest entry
    first; then per merged tile first token, token count, first slot, number of parts."""

    __slots__ = ("table", "entries", "merges", "slots")

    def __init__(self, table, entries, merges, slots):
        self.table, self.entries, self.merges, self.slots = table, entries, merges, slots


def plan_prefill_parts(row_lens, row_starts, tile_tokens: int, kv_heads: int, part_bytes: int = 64 * 128 * 4):
    """Host part of ``PrefillPartsPlan``: ``(entries, merges)`` as lists of tuples, or None where
    whole tiles do as well. A step takes as long as its deepest tile's chain of key tiles (about 1.2 us
    each for a block on its own) or as long as all key tiles take the chip (about 2.4 us for each
    resident block's), whichever is longer. Where the chain is the longer by far (a short portion
    deep into a long sequence), the keys of tiles deeper than the chip's fair share (all key tiles /
    resident blocks) are cut into equal parts no longer than that share. The parts cost a second
    kernel and ``part_bytes`` written and read per part and KV head, so whole tiles stay unless the
    shorter chain saves half as much again as that (measured: one 2,048-token prompt is slower in
    parts, a 512-token portion behind 16,000 cached tokens a quarter faster)."""
    tiles = []
    t = 0
    for n, s in zip(row_lens, row_starts):
        if n > 1:
            for a in range(0, n, tile_tokens):
                c = min(tile_tokens, n - a)
                tiles.append(((s + a + c - 1) // PREFILL_KEY_TILE + 1, t + a, c))
        t += n
    if not tiles or len(tiles) * kv_heads >= 2 * PREFILL_RESIDENT_BLOCKS:
        return None
    total = sum(d for d, _, _ in tiles) * kv_heads
    share = max(PREFILL_MIN_PART, -(-total // PREFILL_RESIDENT_BLOCKS))
    deepest = max(d for d, _, _ in tiles)
    if deepest <= share:
        return None
    slots = sum(-(-d // share) for d, _, _ in tiles if d > share)
    busy_us = 2.4 * total / PREFILL_RESIDENT_BLOCKS
    saved_us = 1.2 * deepest - max(1.2 * share, busy_us)
    cost_us = PREFILL_PARTS_LAUNCH_US + 2 * slots * kv_heads * part_bytes / 3e6
    if saved_us <= PREFILL_PARTS_MARGIN * cost_us:
        return None
    entries, merges, slot = [], [], 0
    for depth, first, count in tiles:
        parts = -(-depth // share)
        if parts == 1:
            entries.append((first, count, 0, depth, -1))
            continue
        per = -(-depth // parts)
        parts = -(-depth // per)
        merges.append((first, count, slot, parts))
        for p in range(parts):
            entries.append((first, count, p * per, min(depth, (p + 1) * per), slot))
            slot += 1
    entries.sort(key=lambda e: e[2] - e[3])  # most key tiles first
    return entries, merges


def _prefill_parts_plan(batch, tile_tokens: int, kv_heads: int, part_bytes: int):
    memo = getattr(batch, "memo", None)
    key = ("prefill_parts", tile_tokens, kv_heads, part_bytes)
    if memo is not None and key in memo:
        return memo[key]
    plan = None
    made = plan_prefill_parts(batch.row_lens, batch.row_starts_host, tile_tokens, kv_heads, part_bytes)
    if made is not None:
        entries, merges = made
        flat = [e[i] for i in range(5) for e in entries] + [m[i] for i in range(4) for m in merges]
        table = torch.tensor(flat, dtype=I32).to(batch.positions.device, non_blocking=True)
        plan = PrefillPartsPlan(table, len(entries), len(merges), sum(m[3] for m in merges))
    if memo is not None:
        memo[key] = plan
    return plan



# ------------------------------------------------------------------------------------- further norms


def layernorm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, eps: float, out_dtype,
              rows: torch.Tensor | None = None) -> torch.Tensor:
    """``(x - mean) / sqrt(var + eps) * weight + bias`` over the float32 rows of ``x`` (all, or those named by
    ``rows``), statistics in float32, the variance being the mean of the squared deviations."""
    _dev(x, "x", F32, 2)
    _dev(weight, "weight", (F32, BF16), 1)
    if weight.shape[0] != x.shape[1]:
        raise ValueError(f"norm weight has {weight.shape[0]} elements for width {x.shape[1]}")
    if bias is not None:
        _dev(bias, "bias", weight.dtype, 1)
        if bias.shape[0] != x.shape[1]:
            raise ValueError(f"norm bias has {bias.shape[0]} elements for width {x.shape[1]}")
    if out_dtype not in (F32, BF16):
        raise TypeError(f"unsupported output dtype {out_dtype}")
    n = x.shape[0]
    if rows is not None:
        _dev(rows, "rows", I32, 1)
        n = rows.shape[0]
    out = torch.empty((n, x.shape[1]), dtype=out_dtype, device=x.device)
    _check(library().ms_layernorm(x.data_ptr(), weight.data_ptr(), _ptr(bias), int(weight.dtype == BF16), out.data_ptr(),
                                  int(out_dtype == BF16), _ptr(rows), n, x.shape[1], float(eps), _stream()), "layernorm")
    return out


GATE_ACTIVATIONS = {"sigmoid": 0, "silu": 1}  # what a gate goes through before it multiplies a normed output


def group_rmsnorm_gate(x: torch.Tensor, group: int, weight: torch.Tensor | None, gate: torch.Tensor | None, eps: float,
                       out_dtype, gate_activation: str = "sigmoid") -> torch.Tensor:
    """``x / rms(group of x) * weight * act(gate)`` for float32 ``x [T, N]`` cut into groups of ``group``
    consecutive elements (``group == N``: one norm over the row). ``weight [N]`` and ``gate`` (float32 ``[T, N]``,
    may be a column slice of a wider matrix) are optional; ``gate_activation``: ``"sigmoid"`` or ``"silu"``."""
    if gate_activation not in GATE_ACTIVATIONS:
        raise NotImplementedError(f"gate activation {gate_activation!r}: the kernel knows {sorted(GATE_ACTIVATIONS)}")
    _dev(x, "x", F32, 2)
    t, n = x.shape
    if group < 1 or n % group:
        raise ValueError(f"a row of {n} elements cannot be cut into groups of {group}")
    if weight is not None:
        _dev(weight, "weight", (F32, BF16), 1)
        if weight.shape[0] != n:
            raise ValueError(f"norm weight has {weight.shape[0]} elements for width {n}")
    gate_stride = 0
    if gate is not None:
        if not (gate.is_cuda and gate.dtype == F32 and gate.dim() == 2 and gate.shape == x.shape and gate.stride(1) == 1):
            raise ValueError("gate must be a float32 matrix of x's shape on the GPU with unit column stride")
        gate_stride = gate.stride(0)
    if out_dtype not in (F32, BF16):
        raise TypeError(f"unsupported output dtype {out_dtype}")
    out = torch.empty((t, n), dtype=out_dtype, device=x.device)
    _check(library().ms_group_rmsnorm_gate(x.data_ptr(), _ptr(weight), int(weight is not None and weight.dtype == BF16), _ptr(gate),
                                           gate_stride, out.data_ptr(), int(out_dtype == BF16), t, n // group, group, float(eps),
                                           GATE_ACTIVATIONS[gate_activation], _stream()), "group_rmsnorm_gate")
    return out


def normed_mean_add(residual: torch.Tensor, streams, weights, eps: float, coef: float) -> None:
    """``residual += coef * sum_i rmsnorm(streams[i]) * weights[i]``: up to four float32 streams of the residual's
    shape, each normed over the row with its own weight."""
    _dev(residual, "residual", F32, 2)
    n = len(streams)
    if not 1 <= n <= 4 or len(weights) != n:
        raise ValueError("one to four streams, each with a weight, are needed")
    for s_, w in zip(streams, weights):
        _dev(s_, "stream", F32, 2)
        _dev(w, "weight", weights[0].dtype, 1)
        if s_.shape != residual.shape or w.shape[0] != residual.shape[1]:
            raise ValueError("streams and weights must have the residual's shape and width")
    _dev(weights[0], "weight", (F32, BF16), 1)
    sp = (ctypes.c_void_p * n)(*[s_.data_ptr() for s_ in streams])
    wp = (ctypes.c_void_p * n)(*[w.data_ptr() for w in weights])
    _check(library().ms_normed_mean_add(residual.data_ptr(), sp, wp, int(weights[0].dtype == BF16), n, residual.shape[0],
                                        residual.shape[1], float(eps), float(coef), _stream()), "normed_mean_add")


def normed_add(residual: torch.Tensor, stream: torch.Tensor | None, weight: torch.Tensor, eps: float, pending: SplitSum | None = None,
               next_out: torch.Tensor | None = None, clear: bool = False) -> None:
    """``residual += rmsnorm(stream + pending) * weight`` row by row: one float32 stream of the residual's shape (None:
    zero) and the partial sums its last matrix product may have left (summed inside the kernel, no kernel of their own).
    ``next_out`` (bfloat16, the residual's shape) receives the new residual rounded, for the next reader that wants it in
    16 bits; with ``clear`` the stream is left zero."""
    if pending is None and stream is None:
        raise ValueError("neither a stream nor a pending sum")
    if pending is None and next_out is None and not clear:
        return normed_mean_add(residual, [stream], [weight], eps, 1.0)
    _dev(residual, "residual", F32, 2)
    _dev(weight, "weight", (F32, BF16), 1)
    if pending is not None:
        _check_split(pending, "pending", residual.shape)
    if stream is not None:
        _dev(stream, "stream", F32, 2)
        if stream.shape != residual.shape:
            raise ValueError("the stream must have the residual's shape")
    if next_out is not None:
        _dev(next_out, "next_out", BF16, 2)
        if next_out.shape != residual.shape:
            raise ValueError("next_out must have the residual's shape")
    if weight.shape[0] != residual.shape[1]:
        raise ValueError("the weight must have the residual's width")
    _check(library().ms_normed_add_pending(residual.data_ptr(), _ptr(stream), pending.parts.data_ptr() if pending is not None else None,
                                           pending.splits if pending is not None else 0, pending.stride if pending is not None else 0,
                                           weight.data_ptr(), int(weight.dtype == BF16), residual.shape[0], residual.shape[1], float(eps),
                                           _ptr(next_out), int(clear), _stream()), "normed_add_pending")


def scale_(x: torch.Tensor, factor: float) -> torch.Tensor:
    """``x *= factor`` in place (float32)."""
    _dev(x, "x", F32)
    _check(library().ms_scale(x.data_ptr(), x.numel(), float(factor), _stream()), "scale")
    return x


def qkv_norm_rope_store(qkv, slots, q_weight, k_weight, eps, rope, k_cache, v_cache, num_heads, num_kv_heads, head_dim,
                        value_dim, out_dtype, pairing: str = "halves", bias: torch.Tensor | None = None,
                        values_are_keys: bool = False, extra_columns: int = 0) -> torch.Tensor:
    """From float32 ``qkv [T, Hq D + Hkv D + Hkv Dv]`` (and ``extra_columns`` more behind them that are not read here): RMS norm of the whole query part and of the whole key
    part of a token (weights ``[Hq D]`` and ``[Hkv D]``; None: no norm), rotation of the first ``rope.shape[1]``
    elements of each query and key head, in pairs as ``pairing`` names them, by the angles of ``rope`` (a
    ``rope_table`` of these tokens; None: no rotation), keys and values stored into the cache pages at ``slots``
    (skipped when ``slots`` is None). Returns the finished queries ``[T, Hq D]`` in ``out_dtype``.

    ``bias`` (one element per column that is read) is added to the projection first. ``values_are_keys``: the matrix has
    no value columns; a token's values are its keys as projected, bias included, before norm and rotation
    (``value_dim == head_dim``)."""
    _dev(qkv, "qkv", F32, 2)
    t = qkv.shape[0]
    nq, nk = num_heads * head_dim, num_kv_heads * head_dim
    if values_are_keys:
        if value_dim != head_dim:
            raise ValueError(f"values that are the keys have the keys' size {head_dim}, not {value_dim}")
        width, v_col = nq + nk, nq
    else:
        width, v_col = nq + nk + num_kv_heads * value_dim, nq + nk
    if extra_columns < 0 or qkv.shape[1] != width + extra_columns:
        raise ValueError(f"qkv has width {qkv.shape[1]}, expected {width + extra_columns}")
    if out_dtype not in (F32, BF16):
        raise TypeError(f"unsupported output dtype {out_dtype}")
    w_bf16 = None
    if (q_weight is None) != (k_weight is None):
        raise ValueError("the query and the key norm come together or not at all")
    if q_weight is not None:
        for w, nm, n in ((q_weight, "q_norm", nq), (k_weight, "k_norm", nk)):
            _dev(w, nm, (F32, BF16), 1)
            if w.shape[0] != n:
                raise ValueError(f"{nm} weight has {w.shape[0]} elements, expected {n}")
        if q_weight.dtype != k_weight.dtype:
            raise TypeError("q_norm and k_norm weights differ in dtype")
        w_bf16 = int(q_weight.dtype == BF16)
    if bias is not None:
        _dev(bias, "bias", (F32, BF16), 1)
        if bias.shape[0] != width:
            raise ValueError(f"the bias has {bias.shape[0]} elements for {width} columns")
        if w_bf16 is not None and int(bias.dtype == BF16) != w_bf16:
            raise TypeError("the bias and the norm weights differ in dtype")
        w_bf16 = int(bias.dtype == BF16)
    page_size = 1
    if slots is not None:
        _dev(slots, "slots", I32, 1)
        if slots.shape[0] != t:
            raise ValueError("one slot per token is needed")
        page_size = _check_caches(k_cache, v_cache, out_dtype, num_kv_heads, head_dim, value_dim)
    rot_dim, pair = 0, _pairing(pairing)
    if rope is not None:
        _dev(rope, "rope", F32, 2)
        rot_dim = rope.shape[1]
        if rope.shape[0] != t or rot_dim % 2 or rot_dim > head_dim or rot_dim < 2:
            raise ValueError(f"rotation table is {tuple(rope.shape)}; {t} tokens and an even width up to {head_dim} are needed")
    q_out = torch.empty((t, nq), dtype=out_dtype, device=qkv.device)
    _check(library().ms_qkv_norm_rope_store(
        qkv.data_ptr(), qkv.shape[1], q_out.data_ptr(), int(out_dtype == BF16), _ptr(slots), _ptr(q_weight), _ptr(k_weight), _ptr(bias),
        v_col, int(w_bf16 or 0), float(eps), _ptr(rope), int(rot_dim), pair, _ptr(k_cache) if slots is not None else None,
        _ptr(v_cache) if slots is not None else None, t, num_heads, num_kv_heads, head_dim, int(value_dim), page_size, _stream()),
        "qkv_norm_rope_store")
    return q_out


HEAD_NORMS = {None: 0, "before": 1, "after": 2}  # where a per-head RMS norm sits relative to the rotation (MS_NORM_* in csrc/attention_prep.hip)
PREPARE_MAX_HEAD_DIM = 1024


def head_prepare_store(qkv, slots, norm: str | None, q_weight, k_weight, eps, rope, pairing, k_cache, v_cache, num_heads,
                       num_kv_heads, head_dim, value_dim, out_dtype, v_first=None, blend: float = 0.0) -> torch.Tensor:
    """From float32 ``qkv [T, Hq D + Hkv D + Hkv Dv]``: rotation of the first ``rope.shape[1]`` elements of each query and
    key head, in pairs as ``pairing`` names them, by the angles of ``rope`` (a ``rope_table`` of these tokens; None: no
    rotation), and an RMS norm per head, ``norm="before"`` the rotation or ``"after"`` it (weights ``[D]`` each, or None for
    a bare division by the root mean square; ``norm=None``: no norm). ``v_first`` (a float32 tensor of at least ``Hkv Dv``
    columns, one row per token, possibly a view of wider rows): the values become ``(1 - blend) v + blend v_first``. Keys
    and values are stored into the cache pages at ``slots`` (skipped when ``slots`` is None). Returns the finished queries
    ``[T, Hq D]`` in ``out_dtype``."""
    _dev(qkv, "qkv", F32, 2)
    t = qkv.shape[0]
    width = num_heads * head_dim + num_kv_heads * (head_dim + value_dim)
    if qkv.shape[1] != width:
        raise ValueError(f"qkv has width {qkv.shape[1]}, expected {width}")
    if out_dtype not in (F32, BF16):
        raise TypeError(f"unsupported output dtype {out_dtype}")
    if norm not in HEAD_NORMS:
        raise ValueError(f"norm {norm!r}: one of {list(HEAD_NORMS)}")
    if max(head_dim, value_dim) > PREPARE_MAX_HEAD_DIM or min(head_dim, value_dim) < 1:
        raise ValueError(f"head sizes {head_dim} / {value_dim} are outside the kernel's range 1..{PREPARE_MAX_HEAD_DIM}")
    w_bf16 = 0
    if (q_weight is None) != (k_weight is None) or (q_weight is not None and norm is None):
        raise ValueError("the query and the key norm's weights come together, and only with a norm")
    if q_weight is not None:
        for w, nm in ((q_weight, "q_norm"), (k_weight, "k_norm")):
            _dev(w, nm, (F32, BF16), 1)
            if w.shape[0] != head_dim:
                raise ValueError(f"{nm} weight has {w.shape[0]} elements for head_dim {head_dim}")
        if q_weight.dtype != k_weight.dtype:
            raise TypeError("q_norm and k_norm weights differ in dtype")
        w_bf16 = int(q_weight.dtype == BF16)
    page_size = 1
    if slots is not None:
        _dev(slots, "slots", I32, 1)
        if slots.shape[0] != t:
            raise ValueError("one slot per token is needed")
        page_size = _check_caches(k_cache, v_cache, out_dtype, num_kv_heads, head_dim, value_dim)
    rot_dim, pair = 0, _pairing(pairing)
    if rope is not None:
        _dev(rope, "rope", F32, 2)
        rot_dim = rope.shape[1]
        if rope.shape[0] != t or rot_dim % 2 or rot_dim > head_dim or rot_dim < 2:
            raise ValueError(f"rotation table is {tuple(rope.shape)}; {t} tokens and an even width up to {head_dim} are needed")
    first_ld = 0
    if v_first is not None:
        if not (isinstance(v_first, torch.Tensor) and v_first.is_cuda and v_first.dtype == F32 and v_first.dim() == 2
                and v_first.stride(1) == 1):
            raise TypeError("v_first must be float32 rows on the GPU with contiguous elements")
        if v_first.shape[0] != t or v_first.shape[1] < num_kv_heads * value_dim:
            raise ValueError(f"v_first is {tuple(v_first.shape)}; {t} rows of at least {num_kv_heads * value_dim} values are needed")
        first_ld = v_first.stride(0)
    q_out = torch.empty((t, num_heads * head_dim), dtype=out_dtype, device=qkv.device)
    _check(library().ms_head_prepare_store(
        qkv.data_ptr(), qkv.shape[1], q_out.data_ptr(), int(out_dtype == BF16), _ptr(slots), _ptr(q_weight), _ptr(k_weight), w_bf16,
        HEAD_NORMS[norm], float(eps), _ptr(rope), int(rot_dim), pair, _ptr(v_first), int(first_ld), float(blend),
        _ptr(k_cache) if slots is not None else None, _ptr(v_cache) if slots is not None else None, t, num_heads, num_kv_heads,
        head_dim, int(value_dim), page_size, _stream()), "head_prepare_store")
    return q_out


# ------------------------------------------------------------------------------------- between projection and attention


def conv_norm_store(x, conv_weight, taps: int, state, batch, q_weight, k_weight, eps, slots, k_cache, v_cache, q_groups: int,
                    k_groups: int, value_heads: int, head_dim: int, value_dim: int, out_dtype) -> torch.Tensor:
    """A short causal convolution over time on every channel of the float32 projection ``x [T, q_groups D + k_groups D +
    value_heads Dv]`` (``conv_weight [channels, taps]``; ``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``, zero before a
    sequence's start), an RMS norm over every group of ``D`` query and key channels (weights ``[D]``, shared by the
    groups; None: no norm), then the store: keys ``[pages, k_groups, page, D]`` and values ``[pages, value_heads, Dv,
    page]`` at ``slots``. Returns the queries ``[T, q_groups D]`` in ``out_dtype``.

    ``state`` (float32 ``[slots + 1, taps - 1, channels]``) holds each request's last ``taps - 1`` projection rows:
    row ``batch.state_slots[b]`` feeds the positions before this step and is brought up to date afterwards. A request
    that starts at position 0 reads nothing of it."""
    _dev(x, "x", F32, 2)
    t = x.shape[0]
    channels = (q_groups + k_groups) * head_dim + value_heads * value_dim
    if x.shape[1] != channels:
        raise ValueError(f"x has width {x.shape[1]}, expected {channels}")
    if out_dtype not in (F32, BF16):
        raise TypeError(f"unsupported output dtype {out_dtype}")
    _dev(conv_weight, "conv_weight", (F32, BF16), 2)
    if tuple(conv_weight.shape) != (channels, taps) or taps < 1:
        raise ValueError(f"conv_weight is {tuple(conv_weight.shape)}, expected [{channels}, {taps}]")
    if (q_weight is None) != (k_weight is None):
        raise ValueError("the query and the key norm come together or not at all")
    for w, nm in ((q_weight, "q_norm"), (k_weight, "k_norm")):
        if w is not None:
            _dev(w, nm, conv_weight.dtype, 1)
            if w.shape[0] != head_dim:
                raise ValueError(f"{nm} weight has {w.shape[0]} elements, expected {head_dim}")
    if taps > 1:
        _dev(state, "state", F32, 3)
        if tuple(state.shape[1:]) != (taps - 1, channels):
            raise ValueError(f"state is {tuple(state.shape)}, expected [slots, {taps - 1}, {channels}]")
    _dev(slots, "slots", I32, 1)
    for name in ("token_row", "positions"):
        _dev(getattr(batch, name), name, I32, 1)
        if getattr(batch, name).shape[0] != t:
            raise ValueError("batch metadata does not match the number of tokens")
    if slots.shape[0] != t or batch.row_start.shape[0] < batch.num_rows + 1:
        raise ValueError("one slot per token and one start per row are needed")
    page = _check_special_caches(k_cache, v_cache, out_dtype, k_groups, head_dim, value_dim, k_groups // value_heads, False)
    q_out = torch.empty((t, q_groups * head_dim), dtype=out_dtype, device=x.device)
    _check(library().ms_conv_norm_store(
        x.data_ptr(), x.shape[1], conv_weight.data_ptr(), int(conv_weight.dtype == BF16), int(taps), _ptr(state) if taps > 1 else None,
        batch.state_slots.data_ptr(), batch.token_row.data_ptr(), batch.positions.data_ptr(), batch.row_start.data_ptr(),
        batch.starts.data_ptr(), _ptr(q_weight), _ptr(k_weight), float(eps), q_out.data_ptr(), slots.data_ptr(), k_cache.data_ptr(),
        v_cache.data_ptr(), int(out_dtype == BF16), t, batch.num_rows, q_groups, k_groups, value_heads, head_dim, value_dim, page,
        _stream()), "conv_norm_store")
    return q_out


def map_difference_norm(a: torch.Tensor, groups: int, per_group: int, value_dim: int, weight: float, eps: float,
                        out_scale: float, out_dtype=None) -> torch.Tensor:
    """``a [T, groups * 2 * per_group * Dv]`` holds two attention maps' outputs per head, ordered (group, map, head of
    the group). Per head: ``o = a1 - weight * a2``, divided by its root mean square over ``Dv`` (``eps`` inside the
    root), times ``out_scale``. Returns ``[T, groups * per_group * Dv]`` in ``out_dtype`` (default: ``a``'s), float32
    arithmetic. The difference of two close maps loses what their rounding lost: give ``a`` in float32."""
    _dev(a, "a", (F32, BF16), 2)
    if a.shape[1] != groups * 2 * per_group * value_dim:
        raise ValueError(f"a has width {a.shape[1]}, expected {groups * 2 * per_group * value_dim}")
    out_dtype = a.dtype if out_dtype is None else out_dtype
    if out_dtype not in (F32, BF16) or (a.dtype == BF16 and out_dtype != BF16):
        raise TypeError(f"unsupported dtypes {a.dtype} -> {out_dtype}")
    out = torch.empty((a.shape[0], groups * per_group * value_dim), dtype=out_dtype, device=a.device)
    _check(library().ms_map_difference_norm(a.data_ptr(), out.data_ptr(), int(a.dtype == BF16), int(out_dtype == BF16), a.shape[0],
                                            groups, per_group, value_dim, float(weight), float(eps), float(out_scale), _stream()),
           "map_difference_norm")
    return out


def latent_prepare(x, q_col: int, kv_col: int | None, rope, rot: int, pairing: str, latent_weight, eps, slots, k_cache, v_cache,
                   heads: int, plain_dim: int, rot_dim: int, latent_dim: int, out_dtype):
    """From the float32 projection ``x``: every head's plain query part into ``q_plain [T, H Dn]``, its turned part into
    the last ``R`` columns of that head in ``q_full [T, H (C + R)]`` (the first ``C`` are left for the caller), and, with
    ``kv_col``, the token's cache row ``[C + R]`` at ``slots`` (``k_cache [pages, 1, page, C + R]``): the latent after an
    RMS norm (``latent_weight``) and the turned shared key part; the normed latent goes to ``v_cache [pages, 1, C, page]``
    as well, as the token's value. The first ``rot`` of the ``R`` elements turn by ``rope``'s angles. Returns
    ``(q_plain, q_full)``."""
    _dev(x, "x", F32, 2)
    t = x.shape[0]
    if out_dtype not in (F32, BF16):
        raise TypeError(f"unsupported output dtype {out_dtype}")
    if rot:
        _dev(rope, "rope", F32, 2)
        if tuple(rope.shape) != (t, rot):
            raise ValueError(f"rotation table is {tuple(rope.shape)}, expected [{t}, {rot}]")
    w_bf16 = 0
    if kv_col is not None:
        _dev(slots, "slots", I32, 1)
        page = _check_special_caches(k_cache, v_cache, out_dtype, 1, latent_dim + rot_dim, latent_dim, 1, False)
        _dev(latent_weight, "latent_weight", (F32, BF16), 1)
        if slots.shape[0] != t or latent_weight.shape[0] != latent_dim:
            raise ValueError("one slot per token and a weight of C elements are needed")
        w_bf16 = int(latent_weight.dtype == BF16)
    q_plain = torch.empty((t, heads * plain_dim), dtype=out_dtype, device=x.device)
    q_full = torch.empty((t, heads * (latent_dim + rot_dim)), dtype=out_dtype, device=x.device)
    _check(library().ms_latent_prepare(
        x.data_ptr(), x.shape[1], int(q_col), -1 if kv_col is None else int(kv_col), _ptr(rope) if rot else None, int(rot),
        _pairing(pairing), _ptr(latent_weight) if kv_col is not None else None, w_bf16, float(eps), q_plain.data_ptr(),
        q_full.data_ptr(), _ptr(slots) if kv_col is not None else None, _ptr(k_cache) if kv_col is not None else None,
        _ptr(v_cache) if kv_col is not None else None, page if kv_col is not None else 1, int(out_dtype == BF16), t, heads, plain_dim,
        rot_dim, latent_dim, _stream()), "latent_prepare")
    return q_plain, q_full


def head_gate_(o: torch.Tensor, x: torch.Tensor, col: int, heads: int) -> torch.Tensor:
    """``o[t, h, :] *= sigmoid(x[t, col + h])`` in place: ``o [T, heads * E]``, ``x`` float32."""
    _dev(o, "o", (F32, BF16), 2)
    _dev(x, "x", F32, 2)
    if o.shape[0] != x.shape[0] or o.shape[1] % heads or x.shape[1] < col + heads:
        raise ValueError("o and x must have the same rows, and x one gate column per head")
    _check(library().ms_head_gate(o.data_ptr(), int(o.dtype == BF16), x.data_ptr(), x.shape[1], int(col), o.shape[0], heads,
                                  o.shape[1] // heads, _stream()), "head_gate")
    return o


def activate(x: torch.Tensor, activation: str, out_dtype) -> torch.Tensor:
    """``act(x)`` elementwise for a feed-forward without a gate: float32 in, ``out_dtype`` out, float32 arithmetic."""
    _dev(x, "x", F32)
    if activation not in ACTIVATIONS or activation in ACTIVATIONS_WITH_LIMIT:
        raise NotImplementedError(f"activation {activation!r} has no ungated form here")
    if out_dtype not in (F32, BF16):
        raise TypeError(f"unsupported output dtype {out_dtype}")
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    _check(library().ms_activate(x.data_ptr(), out.data_ptr(), int(out_dtype == BF16), x.numel(), ACTIVATIONS[activation], _stream()),
           "activate")
    return out


def head_linear(x: torch.Tensor, weights: torch.Tensor, out: torch.Tensor, out_col: int = 0, gate=None) -> torch.Tensor:
    """A matrix product per head: ``out[:, h * stride + out_col : ... + N] = x[:, h * K : (h + 1) * K] @ weights[h]^T`` with
    ``x [M, H K]``, ``weights [H, N, K]`` and ``out [M, H stride]`` (``stride = out.shape[1] / H >= out_col + N``; the other
    columns of ``out`` stay). bfloat16 weights with ``K`` a multiple of 8: one launch of a matrix-core kernel for all
    heads. float32 weights: the true 32-bit product, one launch per head over strided rows. Other sizes: head by head
    through contiguous copies. ``gate = (g, col)``: head ``h``'s results of row ``m`` are multiplied by
    ``sigmoid(g[m, col + h])`` (``g`` float32; ``out_col`` 0 and ``N`` the head's whole stride): in the matrix-core
    kernel's epilogue, else by ``head_gate_`` behind the products."""
    _dev(x, "x", (F32, BF16), 2)
    _dev(weights, "weights", (F32, BF16), 3)
    _dev(out, "out", (F32, BF16), 2)
    h, n, k = weights.shape
    m = x.shape[0]
    if x.shape[1] != h * k or out.shape[0] != m or out.shape[1] % h or out.shape[1] // h < out_col + n:
        raise ValueError(f"head_linear: x {tuple(x.shape)}, weights {tuple(weights.shape)}, out {tuple(out.shape)} at column {out_col}")
    if m == 0:
        return out
    stride = out.shape[1] // h
    lib = library()
    if gate is not None:
        g, g_col = gate
        _dev(g, "gate", F32, 2)
        if g.shape[0] != m or g.shape[1] < g_col + h or out_col != 0 or stride != n:
            raise ValueError("a gate needs one float32 column per head and products that fill their heads' columns")
        if not (weights.dtype == BF16 and k % 8 == 0):
            head_linear(x, weights, out, out_col)
            return head_gate_(out, g, g_col, h)
    if weights.dtype == F32:
        xa = cast(x, F32)
        for i in range(h):
            _check(lib.ms_gemm_f32(xa.data_ptr() + i * k * 4, weights.data_ptr() + i * n * k * 4,
                                   out.data_ptr() + (i * stride + out_col) * out.element_size(), 0 if out.dtype == F32 else 2, m, n, k,
                                   h * k, out.shape[1], _stream()), "gemm_f32")
        return out
    xa = cast(x, BF16)
    if k % 8 == 0:
        _check(lib.ms_head_gemm_bf16(xa.data_ptr(), h * k, weights.data_ptr(), out.data_ptr(), out.shape[1], stride, int(out_col),
                                     int(out.dtype == F32), m, h, n, k, gate[0].data_ptr() if gate is not None else None,
                                     gate[0].shape[1] if gate is not None else 0, int(gate[1]) if gate is not None else 0, _stream()),
               "head_gemm_bf16")
        return out
    for i in range(h):
        y = linear(xa[:, i * k : (i + 1) * k].contiguous(), weights[i], out_dtype=out.dtype)
        out[:, i * stride + out_col : i * stride + out_col + n].copy_(y)
    return out


# ------------------------------------------------------------------------------------- linear recurrences

DECODE_GENERIC_WAVES = 16  # waves that share a (token, head) in the float32 attention of single-token rows (8 or 16)

RECURRENCE_MODES = {"decay": 0, "exp_gates": 1, "wkv": 2}
RECURRENCE_MAX_DIM = 256
RECURRENCE_CHUNKED_FROM = 16  # tokens of the longest row from which a step runs the chunked kernels
WKV_CHUNKED_FROM = 16  # ... and from which the recurrence with a decay per channel does


def gated_recurrence(x: torch.Tensor, columns: dict, heads: int, dim: int, value_dim: int, batch, state: dict, *,
                     mode: str, activation: str | None = None, q_scale: float = 1.0, decay: torch.Tensor | None = None,
                     cap: float = 0.0, i_bias: torch.Tensor | None = None, f_bias: torch.Tensor | None = None,
                     chunks: bool = True, channel_decay: torch.Tensor | None = None, bonus: torch.Tensor | None = None,
                     rows_below: int = 0) -> torch.Tensor:
    """A linear recurrence over a matrix state per (request, head): ``S_t = a_t S_(t-1) + b_t k_t v_t^T``,
    ``o_t = S_t^T q_t``, for the step's rows (``batch.row_start``, ``batch.starts``, ``batch.state_slots``), in float32.

    ``x``: float32 ``[T, ld]`` whose columns hold the projections; ``columns``: first column of ``q`` and ``k``
    (``heads * dim`` wide each), ``v`` (``heads * value_dim``) and, for ``mode="exp_gates"``, ``i`` and ``f`` (``heads``
    each). ``activation`` (None or ``"silu"``) is applied to q, k and v; q is then scaled by ``q_scale``.
    ``mode="decay"``: ``a = decay[head]``, ``b = 1``. ``mode="exp_gates"``: capped exponential gates with a running
    maximum and a normaliser (the kernel's source states the formulas); ``state`` then also holds ``n`` and ``m``.
    ``mode="wkv"``: a decay per key channel and token, given by its logarithm ``channel_decay`` (float32
    ``[T, heads * dim]``, at most zero), and a ``bonus`` (float32 ``[heads, dim]``) for the current token alone:
    ``o_t = (S_(t-1) + diag(bonus) k_t v_t^T)^T q_t``, then ``S_t = diag(exp(channel_decay_t)) S_(t-1) + k_t v_t^T``
    (``dim == value_dim``). Rows of ``WKV_CHUNKED_FROM`` tokens or more run in chunks (head sizes up to 64).
    ``state["S"]``: float32 ``[slots, heads, dim, value_dim]``; rows with ``starts == 0`` begin from zero.
    Returns float32 ``[T, heads * value_dim]``.

    ``rows_below``: ``x`` is the top ``T`` rows of a matrix that has so many rows more (one product of stacked inputs against
    stacked weights leaves each projection in a block of rows of its own); a column number may then count on past the row's
    end into those rows (column ``j * T * ld + c`` is column ``c`` of the row ``j T`` rows further down). Token-by-token
    kernel only.

    Two kernel families compute the same thing: one walks a row's tokens in order with the state in registers (decode
    steps, short portions, head sizes above 128); the other works in chunks of 64 tokens (three passes: each chunk's own
    contribution, a scan over the chunks, each chunk's outputs) and runs when the step's longest row has at least
    ``RECURRENCE_CHUNKED_FROM`` tokens. They differ by the order of float32 sums only. ``chunks=False`` keeps to the
    first (the chunked kernels take the decays' logarithms: a decay of zero has none)."""
    _dev(x, "x", F32, 2)
    t, ld = x.shape
    if mode not in RECURRENCE_MODES:
        raise NotImplementedError(f"recurrence mode {mode!r}: the kernels know {sorted(RECURRENCE_MODES)}")
    if activation not in (None, "silu"):
        raise NotImplementedError(f"activation {activation!r} inside the recurrence: None or 'silu'")
    if dim > RECURRENCE_MAX_DIM or value_dim > RECURRENCE_MAX_DIM or min(dim, value_dim, heads) < 1:
        raise ValueError(f"head sizes {dim} / {value_dim} are outside the recurrence kernels' range 1..{RECURRENCE_MAX_DIM}")
    S = state["S"]
    _dev(S, "S", F32, 4)
    if tuple(S.shape[1:]) != (heads, dim, value_dim):
        raise ValueError(f"state S is {tuple(S.shape)}, expected [slots, {heads}, {dim}, {value_dim}]")
    n = m = None
    if mode == "exp_gates":
        n, m = state["n"], state["m"]
        _dev(n, "n", F32, 3)
        _dev(m, "m", F32, 2)
        if tuple(n.shape) != (S.shape[0], heads, dim) or tuple(m.shape) != (S.shape[0], heads):
            raise ValueError("state n / m do not match S")
        if not cap > 0:
            raise ValueError(f"the gates' cap must be positive, not {cap}")
        for b_, nm in ((i_bias, "i_bias"), (f_bias, "f_bias")):
            if b_ is not None:
                _dev(b_, nm, (F32, BF16), 1)
                if b_.shape[0] != heads:
                    raise ValueError(f"{nm} has {b_.shape[0]} elements for {heads} heads")
        if i_bias is not None and f_bias is not None and i_bias.dtype != f_bias.dtype:
            raise TypeError("the gates' biases differ in dtype")
    elif mode == "wkv":
        _dev(channel_decay, "channel_decay", F32, 2)
        _dev(bonus, "bonus", F32, 2)
        if tuple(channel_decay.shape) != (t, heads * dim) or tuple(bonus.shape) != (heads, dim):
            raise ValueError(f"channel_decay {tuple(channel_decay.shape)} / bonus {tuple(bonus.shape)} do not fit {t} tokens of "
                             f"{heads} heads of {dim}")
        if dim != value_dim:
            raise ValueError(f"wkv heads have keys and values of one size, not {dim} / {value_dim}")
    else:
        _dev(decay, "decay", F32, 1)
        if decay.shape[0] != heads:
            raise ValueError(f"decay has {decay.shape[0]} elements for {heads} heads")
    for name, w in (("q", heads * dim), ("k", heads * dim), ("v", heads * value_dim)) + (
            (("i", heads), ("f", heads)) if mode == "exp_gates" else ()):
        c = columns[name]
        if c < 0 or (c % ld) + w > ld or c // ld > rows_below:
            raise ValueError(f"columns of {name!r} ({c} .. {c + w}) lie outside the matrix of width {ld}")
    for v_, nm in ((batch.row_start, "row_start"), (batch.starts, "starts"), (batch.state_slots, "state_slots")):
        _dev(v_, nm, I32, 1)
    rows = batch.num_rows
    if batch.row_start.shape[0] < rows + 1 or batch.starts.shape[0] < rows or batch.state_slots.shape[0] < rows:
        raise ValueError("batch metadata does not match the number of rows")
    if batch.num_tokens != t:
        raise ValueError("one row of x per token of the step is needed")
    out = torch.empty((t, heads * value_dim), dtype=F32, device=x.device)
    bias = i_bias if i_bias is not None else f_bias
    lib = library()
    lens = getattr(batch, "row_lens", None)
    if rows_below:
        if rows_below < 0 or not x.is_contiguous() or x.untyped_storage().nbytes() - x.storage_offset() * 4 < (t + rows_below) * ld * 4:
            raise ValueError(f"x is not the top of a matrix with {rows_below} more rows")
        chunks = False  # the chunked kernels read columns of the row alone
    if mode == "wkv":
        if chunks and lens is not None and max(lens) >= WKV_CHUNKED_FROM and dim <= lib.ms_wkv_chunk_max_dim():
            per = lib.ms_wkv_chunk_tokens()
            n_chunks = sum(-(-n // per) for n in lens)
            U = torch.empty((n_chunks, heads, dim * dim), dtype=F32, device=x.device)
            G = torch.empty((n_chunks, heads, dim), dtype=F32, device=x.device)
            _check(lib.ms_wkv_chunked(x.data_ptr(), ld, columns["q"], columns["k"], columns["v"], heads, dim, channel_decay.data_ptr(),
                                      heads * dim, bonus.data_ptr(), S.data_ptr(), batch.row_start.data_ptr(), batch.starts.data_ptr(),
                                      batch.state_slots.data_ptr(), out.data_ptr(), rows, n_chunks, U.data_ptr(), G.data_ptr(), _stream()),
                   "wkv_chunked")
            return out
        chunks = False
    if (chunks and lens is not None and max(lens) >= RECURRENCE_CHUNKED_FROM
            and max(dim, value_dim) <= lib.ms_gated_recurrence_chunk_max_dim()):
        per = lib.ms_gated_recurrence_chunk_tokens()
        chunks = sum(-(-n // per) for n in lens)
        U = torch.empty((chunks, heads, dim * value_dim), dtype=F32, device=x.device)
        u = torch.empty((chunks, heads, dim), dtype=F32, device=x.device) if mode == "exp_gates" else None
        cs = torch.empty((chunks, heads, 4), dtype=torch.float64, device=x.device)
        _check(lib.ms_gated_recurrence_chunked(
            x.data_ptr(), ld, columns["q"], columns["k"], columns["v"], columns.get("i", 0), columns.get("f", 0), heads, dim, value_dim,
            int(activation == "silu"), RECURRENCE_MODES[mode], float(q_scale), float(cap), _ptr(decay), _ptr(i_bias), _ptr(f_bias),
            int(bias is not None and bias.dtype == BF16), S.data_ptr(), _ptr(n), _ptr(m), batch.row_start.data_ptr(),
            batch.starts.data_ptr(), batch.state_slots.data_ptr(), out.data_ptr(), rows, chunks, U.data_ptr(), _ptr(u), cs.data_ptr(),
            _stream()), "gated_recurrence_chunked")
        return out
    _check(lib.ms_gated_recurrence(
        x.data_ptr(), ld, columns["q"], columns["k"], columns["v"], columns.get("i", 0), columns.get("f", 0), heads, dim, value_dim,
        int(activation == "silu"), RECURRENCE_MODES[mode], float(q_scale), float(cap), _ptr(decay), _ptr(i_bias), _ptr(f_bias),
        int(bias is not None and bias.dtype == BF16), S.data_ptr(), _ptr(n), _ptr(m), batch.row_start.data_ptr(),
        batch.starts.data_ptr(), batch.state_slots.data_ptr(), out.data_ptr(), rows, _ptr(channel_decay), heads * dim, _ptr(bonus),
        _stream()), "gated_recurrence")
    return out


def rotate_columns_(x: torch.Tensor, col: int, heads: int, dim: int, rope: torch.Tensor | None, pairing: str = "halves",
                    scale: float = 1.0) -> torch.Tensor:
    """In place on the float32 ``x [T, ld]``: the ``heads`` heads of ``dim`` elements from column ``col`` on have their
    first ``rope.shape[1]`` elements turned by the angles of ``rope`` (a ``rope_table`` of these tokens; None: no
    rotation), and every element of them is then multiplied by ``scale``."""
    _dev(x, "x", F32, 2)
    t = x.shape[0]
    rot = 0
    if rope is not None:
        _dev(rope, "rope", F32, 2)
        rot = rope.shape[1]
        if rope.shape[0] != t or rot % 2 or rot > dim:
            raise ValueError(f"rotation table is {tuple(rope.shape)}; {t} tokens and an even width up to {dim} are needed")
    if col < 0 or col + heads * dim > x.shape[1]:
        raise ValueError(f"columns {col} .. {col + heads * dim} lie outside the matrix of width {x.shape[1]}")
    if rot == 0 and scale == 1.0:
        return x
    _check(library().ms_rotate_columns(x.data_ptr(), x.shape[1], int(col), t, heads, dim, _ptr(rope), rot, _pairing(pairing), float(scale),
                                       _stream()), "rotate_columns")
    return x


def token_shift_mix(h: torch.Tensor, mu: torch.Tensor, carry: torch.Tensor, batch) -> torch.Tensor:
    """``out[s, t] = h[t] + (h[t - 1] - h[t]) * mu[s]`` for every blend ``s``: ``h [T, W]`` and ``mu [n, W]`` in one dtype,
    the result ``[n, T, W]`` in the same (float32 arithmetic, rounded once). ``h[t - 1]`` of a row's first token is the row
    its request carried in ``carry [slots, W]`` (float32; zeros where the request starts in this step), and the row's last
    token of this step is carried from here on."""
    _dev(h, "h", (F32, BF16), 2)
    _dev(mu, "mu", h.dtype, 2)
    _dev(carry, "carry", F32, 2)
    t, w = h.shape
    if mu.shape[1] != w or carry.shape[1] != w:
        raise ValueError(f"mu {tuple(mu.shape)} / carry {tuple(carry.shape)} do not fit rows of {w}")
    for v_, nm in ((batch.token_row, "token_row"), (batch.row_start, "row_start"), (batch.starts, "starts"), (batch.state_slots, "state_slots")):
        _dev(v_, nm, I32, 1)
    if batch.num_tokens != t or batch.token_row.shape[0] != t:
        raise ValueError("one row of h per token of the step is needed")
    out = torch.empty((mu.shape[0], t, w), dtype=h.dtype, device=h.device)
    _check(library().ms_token_shift_mix(h.data_ptr(), mu.data_ptr(), out.data_ptr(), int(h.dtype == BF16), carry.data_ptr(),
                                        batch.token_row.data_ptr(), batch.row_start.data_ptr(), batch.starts.data_ptr(),
                                        batch.state_slots.data_ptr(), t, w, mu.shape[0], _stream()), "token_shift_mix")
    return out


def channel_decay(a: torch.Tensor, w2: torch.Tensor, w0: torch.Tensor, log: bool = False) -> torch.Tensor:
    """``exp(-exp(tanh(a) @ w2^T + w0))``: float32 ``[T, C]`` from the float32 ``a [T, R]``, ``w2 [C, R]`` (float32: the product
    is the true 32-bit one, a chain of multiply-adds in ascending ``r``) and ``w0 [C]``. ``log``: the decays' logarithms
    ``-exp(...)`` instead (what the recurrence kernels take). Three launches: the tanh, the product, the exponentials."""
    _dev(a, "a", F32, 2)
    _dev(w2, "w2", F32, 2)
    _dev(w0, "w0", (F32, BF16), 1)
    c, r = w2.shape
    if a.shape[1] != r or w0.shape[0] != c:
        raise ValueError(f"a {tuple(a.shape)}, w2 {tuple(w2.shape)} and w0 {tuple(w0.shape)} do not fit")
    z = linear(activate(a, "tanh", F32), w2, out_dtype=F32)
    _check(library().ms_neg_exp_bias(z.data_ptr(), w0.data_ptr(), int(w0.dtype == BF16), z.shape[0], c, int(not log), _stream()), "neg_exp_bias")
    return z

# ------------------------------------------------------------------------------------- sampling


def sample_rows(logits, temperature=None, top_p=None, seed=None, counter=None) -> torch.Tensor:
    """``int32 [rows]`` token ids from float32 ``logits [rows, vocab]``. Without ``temperature`` every
    row takes the first maximal index; with it, rows whose temperature is 0 still do."""
    _dev(logits, "logits", F32, 2)
    rows, vocab = logits.shape
    if temperature is not None:
        _dev(temperature, "temperature", F32, 1)
        _dev(seed, "seed", I32, 1)
        _dev(counter, "counter", I32, 1)
        if top_p is not None:
            _dev(top_p, "top_p", F32, 1)
        for v in (temperature, seed, counter) + ((top_p,) if top_p is not None else ()):
            if v.shape[0] != rows:
                raise ValueError("one sampling parameter per row is needed")
    out = torch.empty((rows,), dtype=I32, device=logits.device)
    lib = library()
    need = lib.ms_sample_scratch_bytes(rows)
    if need < 0:
        raise ValueError(f"sample_rows: {rows} rows are more than one call takes")
    scratch = torch.empty((need,), dtype=torch.uint8, device=logits.device)
    _check(lib.ms_sample_rows(logits.data_ptr(), rows, vocab, vocab, _ptr(temperature), _ptr(top_p), _ptr(seed),
                              _ptr(counter), scratch.data_ptr(), out.data_ptr(), _stream()), "sample_rows")
    return out


def sample_rows_static(logits, out, temperature=None, top_p=None, seed=None, counter=None) -> torch.Tensor:
    """``sample_rows`` into the caller's ``out`` (int32 ``[rows]``) without allocating anything: the
    candidates between the two kernels lie in an array inside the library, one per GPU, instead of
    in a scratch tensor. For callers that cannot allocate (under graph capture, say). At most
    ``ms_sample_rows_static_max_rows()`` rows; calls that overlap on one GPU race for the array."""
    _dev(logits, "logits", F32, 2)
    _dev(out, "out", I32, 1)
    rows, vocab = logits.shape
    if out.shape[0] != rows:
        raise ValueError("one output element per row is needed")
    lib = library()
    most = lib.ms_sample_rows_static_max_rows()
    if rows > most:
        raise ValueError(f"sample_rows_static takes at most {most} rows, got {rows}: use sample_rows")
    if temperature is not None:
        _dev(temperature, "temperature", F32, 1)
        _dev(seed, "seed", I32, 1)
        _dev(counter, "counter", I32, 1)
        if top_p is not None:
            _dev(top_p, "top_p", F32, 1)
        for v in (temperature, seed, counter) + ((top_p,) if top_p is not None else ()):
            if v.shape[0] != rows:
                raise ValueError("one sampling parameter per row is needed")
    _check(lib.ms_sample_rows_static(logits.data_ptr(), rows, vocab, vocab, _ptr(temperature), _ptr(top_p), _ptr(seed),
                                     _ptr(counter), out.data_ptr(), _stream()), "sample_rows_static")
    return out


# ------------------------------------------------------------------------------------- measurement


def measure_read(buffer: torch.Tensor, blocks: int = 4096) -> torch.Tensor:
    """Streams ``buffer`` (contiguous, a multiple of 16 bytes) through ``blocks`` blocks once and
    returns their checksums ``int32 [blocks]``: the read half of the memory system's rate."""
    if not buffer.is_cuda or not buffer.is_contiguous():
        raise ValueError("measure_read takes a contiguous tensor on the GPU")
    out = torch.empty((blocks,), dtype=I32, device=buffer.device)
    _check(library().ms_measure_read(buffer.data_ptr(), buffer.numel() * buffer.element_size(), blocks, out.data_ptr(),
                                     _stream()), "measure_read")
    return out


def measure_copy(src: torch.Tensor, dst: torch.Tensor, blocks: int = 4096) -> None:
    """``dst[:] = src`` as a streaming copy of ``blocks`` blocks (both contiguous, same size, a multiple
    of 16 bytes)."""
    if not (src.is_cuda and dst.is_cuda and src.is_contiguous() and dst.is_contiguous()):
        raise ValueError("measure_copy takes contiguous tensors on the GPU")
    n = src.numel() * src.element_size()
    if n != dst.numel() * dst.element_size():
        raise ValueError("source and destination differ in size")
    _check(library().ms_measure_copy(src.data_ptr(), dst.data_ptr(), n, blocks, _stream()), "measure_copy")
