"""The operations of the engine, each one a hand-written HIP kernel for gfx950.

Every function here checks its operands on the host (device, dtype, shape,
contiguity) and then launches the kernel on the current HIP stream. There is
no CPU path: an operand that is not on a GPU, a missing compiler or a library
that cannot be loaded raise KernelUnavailable. Sizes a kernel cannot take raise
InvalidArgument before anything is launched.
"""

from __future__ import annotations

import ctypes
import functools
from typing import Dict, Optional

import torch

from ..errors import InvalidArgument, KernelUnavailable
from . import build

F32, BF16, F16 = 0, 1, 2
_CODES = {torch.float32: F32, torch.bfloat16: BF16}
_CACHE_CODES = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}

# The cache of keys and values has a precision of its own (the reference's KVCacheConfig.dtype,
# src/kv/paged_kv_cache.h:18-25: float32 arithmetic over a narrower cache is its default arrangement). Per
# compute mode, the cache dtypes some kernel here reads and writes; the first is the mode's default.
CACHE_DTYPES = {"float32": ("float32", "bfloat16", "float16"), "bfloat16": ("bfloat16",)}
_CACHE_DTYPE_NAMES = {"float32": "float32", "fp32": "float32", "f32": "float32", "bfloat16": "bfloat16",
                      "bf16": "bfloat16", "float16": "float16", "fp16": "float16", "f16": "float16"}


def cache_dtype_for(mode: str, asked: Optional[str] = None) -> str:
    """The cache dtype a compute mode runs over: its own by default, ``asked`` if the kernels take the pair."""
    if mode not in CACHE_DTYPES:
        raise InvalidArgument(f"unknown compute mode '{mode}'")
    if asked is None:
        return CACHE_DTYPES[mode][0]
    name = _CACHE_DTYPE_NAMES.get(asked)
    if name is None:
        raise InvalidArgument(f"the cache dtype must be float32, bfloat16 or float16, got '{asked}'")
    if name not in CACHE_DTYPES[mode]:
        raise InvalidArgument(f"no kernel runs {mode} arithmetic over a {name} cache: with --dtype {mode} the cache "
                              f"can be {' or '.join(CACHE_DTYPES[mode])} (the matrix-core attention kernels read "
                              f"bfloat16 pages; float32 arithmetic reads any of the three)")
    return name

_c_int, _c_float, _c_void, _c_long = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_long

# library key -> (file stem, source)
_SOURCES = {
    "elementwise": ("tie_elementwise", "elementwise.hip"),
    "gemm_generic": ("tie_gemm_generic", "gemm_generic.hip"),
    "attention_generic": ("tie_attention_generic", "attention_generic.hip"),
    "skinny_gemm_bf16": ("tie_skinny_gemm_bf16", "skinny_gemm_bf16.hip"),
    "gemm_bf16": ("tie_gemm_bf16", "gemm_bf16.hip"),
    "sample_filtered": ("tie_sample_filtered", "sample_filtered.hip"),
    "machine_peaks": ("tie_machine_peaks", "machine_peaks.hip"),
}
# libraries compiled once per head size: key -> (file stem prefix, source)
_PER_HEAD_DIM = {
    "attention_decode_bf16": ("tie_attention_decode_bf16", "attention_decode_bf16.hip"),
    "attention_prefill_bf16": ("tie_attention_prefill_bf16", "attention_prefill_bf16.hip"),
}
MFMA_HEAD_DIMS = tuple(range(16, 257, 16))   # head sizes the matrix-core attention kernels are built for
MAX_KEY_SPLITS = 256      # MERGE_MAX_SPLITS of csrc/attention_merge.h: the most shares one row's keys are cut into
MAX_HEAD_DIM = 512        # the largest head size any attention kernel takes (the generic ones)
MAX_STEP_TOKENS = 65535   # rows of one step: a grid dimension of the row-wise kernels

_SIGNATURES = {
    "machine_peaks": {
        "tie_stream_read": [_c_void, ctypes.c_longlong, _c_int, _c_void, _c_void, _c_void],
        "tie_mfma_rate": [_c_int, _c_int, _c_void, _c_void, _c_void],
    },
    "sample_filtered": {
        "tie_sample_filtered": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                                _c_int, _c_void, _c_int, _c_int, _c_void],
    },
    "elementwise": {
        "tie_embed": [_c_void, _c_int, _c_void, _c_void, _c_int, _c_int, _c_void],
        "tie_rms_norm": [_c_void, _c_int, _c_void, _c_float, _c_void, _c_int, _c_void, _c_int, _c_int, _c_void],
        "tie_swiglu": [_c_void, _c_int, _c_void, _c_int, _c_int, _c_int, _c_void],
        "tie_cast": [_c_void, _c_int, _c_void, _c_int, ctypes.c_longlong, _c_void],
        "tie_scale_rows": [_c_void, _c_int, _c_int, _c_int, _c_void, _c_int, _c_float, _c_float, _c_void],
        "tie_add_bias": [_c_void, _c_int, _c_int, _c_int, _c_void, _c_void],
        "tie_take_tokens": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_void],
        "tie_random_fill": [_c_void, ctypes.c_longlong, ctypes.c_ulonglong, _c_int, ctypes.c_double, _c_void],
        "tie_rope_angles": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_void],
        "tie_qk_norm_rope_kv_write": [_c_void, _c_int, _c_void, _c_int, _c_void, _c_void, _c_float, _c_void, _c_void,
                                      _c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_void, _c_int, _c_int,
                                      _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_long, _c_int, _c_int, _c_int,
                                      _c_void],
        "tie_add_partials_rms_norm": [_c_void, _c_void, _c_long, _c_int, _c_void, _c_float, _c_void, _c_int, _c_int,
                                      _c_int, _c_void],
        "tie_argmax": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_void],
        "tie_sample": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_int, _c_void, _c_int,
                       _c_int, _c_void],
        "tie_argmax_static": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_void],
    },
    "gemm_generic": {
        "tie_gemm_generic": [_c_void, _c_int, _c_void, _c_int, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int,
                             _c_void],
    },
    "attention_generic": {
        "tie_paged_attention_generic": [_c_void, _c_int, _c_void, _c_void, _c_int, _c_void, _c_int, _c_void, _c_void,
                                        _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                                        _c_int, _c_void],
    },
    "skinny_gemm_bf16": {
        "tie_skinny_gemm_splits": [_c_int, _c_int],
        "tie_skinny_few_rows_plan": [_c_int, _c_int, _c_int, _c_int, _c_void, _c_void],
        "tie_skinny_gemm_bf16_with": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                      _c_int, _c_int, _c_int, _c_void],
        "tie_skinny_gemm_bf16": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                 _c_int, _c_void],
        "tie_skinny_norm_epilogue_rows": [_c_int, _c_int],
        "tie_skinny_gemm_bf16_norm": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                      _c_int, _c_void, _c_int, _c_float, _c_float, _c_void, _c_void, _c_void, _c_int,
                                      _c_int, _c_int, _c_void],
    },
    "gemm_bf16": {
        "tie_gemm_bf16_splits": [_c_int, _c_int, _c_int, _c_int],
        "tie_gemm_bf16_tile": [_c_int, _c_int, _c_int, _c_int, _c_int],
        "tie_gemm_bf16_wins_few_rows": [_c_int, _c_int, _c_int, _c_int, _c_int],
        "tie_gemm_bf16": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                          _c_int, _c_void],
    },
    "attention_prefill_bf16": {
        "tie_attention_prefill_rows_per_item": [_c_int],
        "tie_attention_prefill_bf16": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_int,
                                       _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_void, _c_void,
                                       _c_void, _c_int, _c_void],
        "tie_attention_prefill_bf16_with": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                                            _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_void,
                                            _c_void, _c_void, _c_int, _c_int, _c_void],
    },
    "attention_decode_bf16": {
        "tie_attention_decode_head_dim": [],
        "tie_attention_max_splits": [],
        "tie_attention_decode_bf16": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                                      _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int,
                                      _c_void],
        "tie_attention_decode_prepares": [_c_int],
        "tie_attention_decode_prepared_bf16": [_c_void, _c_long, _c_int, _c_int, _c_void, _c_void, _c_float, _c_void,
                                               _c_int, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                                               _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                                               _c_int, _c_int, _c_void, _c_int, _c_void],
        "tie_attention_decode_bf16_with": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                                           _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int,
                                           _c_int, _c_void, _c_int, _c_void],
    },
}

_libs = {}


def library_list(head_dims=(16, 32, 48, 64, 80, 96, 112, 128, 256)):
    """``(name, source, defines)`` of every library, for building them all up front.

    The per-head-size libraries are listed for ``head_dims``; any other head size is compiled the
    first time a model with it runs.
    """
    libs = [(stem, source, {}) for stem, source in _SOURCES.values()]
    for stem, source in _PER_HEAD_DIM.values():
        for d in head_dims:
            libs.append((f"{stem}_hd{d}", source, {"HEAD_DIM": d}))
    return libs


def _lib(key: str, head_dim: int = 0):
    cache_key = (key, head_dim)
    lib = _libs.get(cache_key)
    if lib is None:
        if head_dim:
            stem, source = _PER_HEAD_DIM[key]
            lib = build.load_library(f"{stem}_hd{head_dim}", source, {"HEAD_DIM": head_dim})
        else:
            stem, source = _SOURCES[key]
            lib = build.load_library(stem, source)
        for fn, argtypes in _SIGNATURES[key].items():
            f = getattr(lib, fn)
            f.argtypes = argtypes
            f.restype = _c_int
        _libs[cache_key] = lib
    return lib


# The current stream's handle, asked for at every launch. torch's public way (a Stream object built anew each time)
# costs several microseconds a call, which at a few hundred launches a step is milliseconds of a prefill step
# that the GPU then waits for; the raw call behind it costs a fraction of one.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    if _raw_stream is not None and _current_device is not None:
        return _raw_stream(_current_device())
    return torch.cuda.current_stream().cuda_stream


_recording: Optional[list] = None     # while a list: every launch is also noted in it, as (function, arguments, name)


def start_recording() -> list:
    """From now on every kernel launch is also noted, as ``(function, arguments, name)``; returns the list."""
    global _recording
    _recording = []
    return _recording


def stop_recording() -> None:
    global _recording
    _recording = None


def _call(fn, what: str, *args) -> None:
    """One kernel launch through the C interface: its status checked, the call noted if launches are being recorded."""
    status = fn(*args)
    if _recording is not None:
        _recording.append((fn, args, what))
    _check(status, what)


def replay_call(fn, what: str, args) -> None:
    """A noted launch again, with the arguments given (see ``models.builder``: layers of one shape)."""
    _check(fn(*args), what)


def _check(status: int, what: str) -> None:
    if status == 0:
        return
    if status < 0:
        raise InvalidArgument(f"{what}: the kernel refused its arguments")
    raise KernelUnavailable(f"{what}: HIP error {status} at launch")


def _gpu(t: torch.Tensor, name: str) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise InvalidArgument(f"{name} must be a tensor")
    if not t.is_cuda:
        raise KernelUnavailable(
            f"{name} is on '{t.device}': the engine's kernels run on a GPU only and have no CPU fallback")
    if not t.is_contiguous():
        raise InvalidArgument(f"{name} must be contiguous")
    return t


def _gpu_strided(t: torch.Tensor, name: str) -> torch.Tensor:
    """A 2-D GPU tensor whose rows are contiguous but may lie further apart than their width."""
    if not isinstance(t, torch.Tensor) or t.dim() != 2:
        raise InvalidArgument(f"{name} must be a 2-D tensor")
    if not t.is_cuda:
        raise KernelUnavailable(
            f"{name} is on '{t.device}': the engine's kernels run on a GPU only and have no CPU fallback")
    if t.stride(1) != 1 or t.stride(0) < t.shape[1]:
        raise InvalidArgument(f"{name} must have contiguous rows")
    return t


def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, KVH: int, block_size: int, Dh: int) -> None:
    """Keys ``[pages, kv heads, block_size, head_dim]``; values transposed in the page ``[pages, kv heads, head_dim, block_size]``."""
    if k_cache.dim() != 4 or v_cache.dim() != 4 or k_cache.dtype != v_cache.dtype or \
            tuple(k_cache.shape[1:]) != (KVH, block_size, Dh) or \
            tuple(v_cache.shape) != (k_cache.shape[0], KVH, Dh, block_size):
        raise InvalidArgument(f"KV cache planes {list(k_cache.shape)} / {list(v_cache.shape)} do not fit "
                              f"{KVH} kv heads, block size {block_size}, head_dim {Dh} "
                              f"(keys [pages, heads, block, dim], values [pages, heads, dim, block])")


def _code(t: torch.Tensor, name: str) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise InvalidArgument(f"{name} must be float32 or bfloat16, got {t.dtype}") from None


def _cache_code(cache: torch.Tensor, beside: torch.Tensor, name: str) -> int:
    """The type code of a cache plane; float16 pages go with float32 activations only."""
    try:
        code = _CACHE_CODES[cache.dtype]
    except KeyError:
        raise InvalidArgument(f"{name} must be float32, bfloat16 or float16, got {cache.dtype}") from None
    if code == F16 and beside.dtype != torch.float32:
        raise InvalidArgument(f"a float16 {name} goes with float32 queries, not {beside.dtype}")
    return code


def _i32(t: torch.Tensor, name: str, numel: Optional[int] = None) -> torch.Tensor:
    _gpu(t, name)
    if t.dtype != torch.int32:
        raise InvalidArgument(f"{name} must be int32, got {t.dtype}")
    if numel is not None and t.numel() < numel:
        raise InvalidArgument(f"{name} holds {t.numel()} entries, {numel} are needed")
    return t


def _f32(t: torch.Tensor, name: str, shape=None) -> torch.Tensor:
    _gpu(t, name)
    if t.dtype != torch.float32:
        raise InvalidArgument(f"{name} must be float32, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise InvalidArgument(f"{name} has shape {list(t.shape)}, expected {list(shape)}")
    return t


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


# --------------------------------------------------------------------- ops
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, :] = float32(table[ids[t], :]); ids must already be checked against the table."""
    _gpu(table, "embedding table")
    T = ids.numel()
    V, D = table.shape
    _i32(ids, "token ids")
    _f32(out, "embedding output", (T, D))
    _call(_lib("elementwise").tie_embed, "embed", table.data_ptr(), _code(table, "embedding table"), ids.data_ptr(),
                                         out.data_ptr(), T, D, _stream())


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
             rows: Optional[torch.Tensor] = None) -> None:
    """out[r] = RMSNorm(x[rows[r]] if rows is given else x[r]) * weight, statistics in float32."""
    _gpu(x, "rms_norm input")
    _gpu(out, "rms_norm output")
    n = x.shape[-1]
    _f32(weight, "rms_norm weight", (n,))
    R = out.numel() // n if n else 0
    if out.shape[-1] != n:
        raise InvalidArgument(f"rms_norm output has width {out.shape[-1]}, input {n}")
    if rows is None:
        if x.numel() != out.numel():
            raise InvalidArgument(f"rms_norm output {list(out.shape)} does not match input {list(x.shape)}")
    else:
        _i32(rows, "rms_norm rows", R)
    _call(_lib("elementwise").tie_rms_norm, "rms_norm", x.data_ptr(), _code(x, "rms_norm input"), weight.data_ptr(), float(eps),
                                            out.data_ptr(), _code(out, "rms_norm output"), _ptr(rows), R, n,
                                            _stream())


def add_partials(x: torch.Tensor, partials: torch.Tensor, weight: Optional[torch.Tensor] = None, eps: float = 0.0,
                 out: Optional[torch.Tensor] = None) -> None:
    """x += partials[0] + partials[1] + ... (float32, in plane order); with ``weight``, out = RMSNorm(x) * weight too.

    ``partials`` is the ``[S, R, n]`` output of a product cut along K (``skinny_gemm_bf16(splits=S)``).
    """
    _gpu(x, "partial sums' target")
    _gpu(partials, "partial sums")
    if x.dtype != torch.float32 or partials.dtype != torch.float32 or partials.dim() != 3 or x.dim() != 2 or \
            tuple(partials.shape[1:]) != tuple(x.shape):
        raise InvalidArgument(f"add_partials: target {list(x.shape)} {x.dtype}, partial sums {list(partials.shape)} "
                              f"{partials.dtype}; both must be float32 and the planes shaped like the target")
    R, n = x.shape
    code = F32
    if weight is not None:
        _f32(weight, "rms_norm weight", (n,))
        _gpu(out, "rms_norm output")
        if tuple(out.shape) != (R, n):
            raise InvalidArgument(f"rms_norm output {list(out.shape)} does not match input {[R, n]}")
        code = _code(out, "rms_norm output")
    _call(_lib("elementwise").tie_add_partials_rms_norm, "add_partials",
        x.data_ptr(), partials.data_ptr(), R * n, partials.shape[0], _ptr(weight), float(eps), _ptr(out), code, R, n,
        _stream())


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i] for gate_up of shape [T, 2I]."""
    _gpu(gate_up, "swiglu input")
    _gpu(out, "swiglu output")
    T, two_i = gate_up.shape
    if two_i % 2 or tuple(out.shape) != (T, two_i // 2):
        raise InvalidArgument(f"swiglu: input {list(gate_up.shape)} and output {list(out.shape)} do not match")
    _call(_lib("elementwise").tie_swiglu, "swiglu", gate_up.data_ptr(), _code(gate_up, "swiglu input"), out.data_ptr(),
                                          _code(out, "swiglu output"), T, two_i // 2, _stream())


def cast(x: torch.Tensor, out: torch.Tensor) -> None:
    _gpu(x, "cast input")
    _gpu(out, "cast output")
    if x.numel() != out.numel():
        raise InvalidArgument("cast: sizes differ")
    _call(_lib("elementwise").tie_cast, "cast", x.data_ptr(), _code(x, "cast input"), out.data_ptr(),
                                        _code(out, "cast output"), x.numel(), _stream())


def take_tokens(tokens: torch.Tensor, sources: torch.Tensor, previous: torch.Tensor) -> None:
    """``tokens[i] = previous[sources[i]]`` where ``sources[i] >= 0`` (all int32 on the device): the rows of a step
    whose token an earlier step's sampling left on the GPU, unread by the host."""
    T = tokens.numel()
    _i32(tokens, "tokens")
    _i32(sources, "token sources", T)
    _i32(previous, "the earlier step's tokens")
    _call(_lib("elementwise").tie_take_tokens, "take_tokens", tokens.data_ptr(), sources.data_ptr(), previous.data_ptr(),
          T, previous.numel(), _stream())


def add_bias(rows: torch.Tensor, bias: torch.Tensor) -> None:
    """rows[m] += bias, in place (float32 arithmetic; rows float32 or bfloat16, bias float32 ``[width]``)."""
    _gpu(rows, "rows")
    if rows.dim() != 2 or not rows.is_contiguous():
        raise InvalidArgument(f"add_bias takes contiguous rows [M, width], got {list(rows.shape)}")
    _f32(bias, "bias", (rows.shape[1],))
    _call(_lib("elementwise").tie_add_bias, "add_bias", rows.data_ptr(), _code(rows, "rows"), rows.shape[0],
          rows.shape[1], bias.data_ptr(), _stream())


def scale_rows(rows: torch.Tensor, row_scale: "RowScale") -> None:
    """``rows[m] *= 1 / sqrt(row_scale.squares[m].sum() / n + eps)`` in place (bfloat16 or float32): for rows that
    were left without their norm's factor and go to a product that cannot apply it."""
    _gpu(rows, "rows")
    M, n = rows.shape
    _f32(row_scale.squares, "sums of squares")
    if row_scale.squares.dim() != 2 or row_scale.squares.shape[0] < M or not row_scale.squares.is_contiguous():
        raise InvalidArgument(f"sums of squares {list(row_scale.squares.shape)} do not cover {M} rows")
    _call(_lib("elementwise").tie_scale_rows, "scale_rows", rows.data_ptr(), _code(rows, "rows"), M, n,
          row_scale.squares.data_ptr(), row_scale.squares.shape[1], float(row_scale.n), float(row_scale.eps), _stream())


def random_fill(out: torch.Tensor, key: int, kind: str, scale: float) -> None:
    """Fills float32 ``out`` with the random weights of the stream ``key``: element i depends on (key, i) alone
    and equals, bit for bit, what ``weights.random_init`` draws on the host. ``kind``: "normal" (``scale`` the
    standard deviation) or "one_plus_uniform" (1 + U(-scale, scale))."""
    _f32(out, "random output")
    if not out.is_contiguous():
        raise InvalidArgument("random_fill needs a contiguous tensor")
    kinds = {"normal": 0, "one_plus_uniform": 1}
    if kind not in kinds:
        raise InvalidArgument(f"random_fill draws 'normal' or 'one_plus_uniform', not '{kind}'")
    if out.numel():
        _call(_lib("elementwise").tie_random_fill, "random_fill", out.data_ptr(), out.numel(), int(key) & (2 ** 64 - 1),
              kinds[kind], float(scale), _stream())


def stream_read(data: torch.Tensor, sink: torch.Tensor, workgroups: int = 2048) -> int:
    """Launches a kernel that reads ``data`` once, in consecutive runs a wave; returns the bytes it reads (whole
    chunks of 8 KB a wave). For measuring what a streaming read of cold memory reaches: the caller times it."""
    _gpu(data, "data")
    _i32(sink, "sink")
    read = ctypes.c_longlong(0)
    _call(_lib("machine_peaks").tie_stream_read, "stream_read", data.data_ptr(), data.numel() * data.element_size(),
          int(workgroups), sink.data_ptr(), ctypes.addressof(read), _stream())
    return int(read.value)


def mfma_rate(sink: torch.Tensor, workgroups: int = 1024, rounds: int = 4096) -> float:
    """Launches a kernel of bfloat16 matrix instructions on registers alone; returns its floating-point operations.
    For measuring the rate the matrix cores sustain: the caller times it."""
    _f32(sink, "sink")
    flops = ctypes.c_double(0.0)
    _call(_lib("machine_peaks").tie_mfma_rate, "mfma_rate", int(workgroups), int(rounds), sink.data_ptr(),
          ctypes.addressof(flops), _stream())
    return float(flops.value)


def gemm_generic(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """out (+)= x @ w.T with float32 multiply-adds; operands float32 or bfloat16 in any mix."""
    _gpu(x, "matmul input")
    _gpu(w, "matmul weight")
    _gpu(out, "matmul output")
    T, K = x.shape
    N, K2 = w.shape
    if K != K2 or tuple(out.shape) != (T, N):
        raise InvalidArgument(f"matmul: input {list(x.shape)}, weight {list(w.shape)}, output {list(out.shape)}")
    _call(_lib("gemm_generic").tie_gemm_generic, "gemm_generic",
        x.data_ptr(), _code(x, "matmul input"), w.data_ptr(), _code(w, "matmul weight"), out.data_ptr(),
        _code(out, "matmul output"), int(accumulate), T, N, K, _stream())


class PackedWeight:
    """A bfloat16 ``[N, K]`` weight stored as ``[N/16][K/32]`` blocks of 1 KB in the matrix cores' operand order.

    Block (t, b) holds rows 16 t .. 16 t + 15 over k = 32 b .. 32 b + 31; within it the 8 elements of
    (row r, k-chunk c) lie at element (16 c + r) * 8. A wave of the decode product then loads 1 KB of
    consecutive memory per matrix instruction and walks K as one contiguous run, and the tiled product
    stages one block per load. Built once at load time by ``pack_weight``; only the bfloat16 products
    read it (``N % 16 == 0`` and ``K % 32 == 0``).
    """

    __slots__ = ("blocks", "shape")
    dtype = torch.bfloat16

    def __init__(self, blocks: torch.Tensor, shape):
        self.blocks = blocks
        self.shape = tuple(shape)

    def data_ptr(self) -> int:
        return self.blocks.data_ptr()

    @property
    def device(self):
        return self.blocks.device

    def unpacked(self) -> torch.Tensor:
        """The ``[N, K]`` row-major matrix again (a copy)."""
        N, K = self.shape
        return self.blocks.view(N // 16, K // 32, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(N, K).contiguous()


def packable(w) -> bool:
    """Whether ``pack_weight`` takes this matrix: bfloat16, on the GPU, rows in steps of 16 and K in steps of 32.

    K between 96 and 2^22 is what the tiled product's packed path takes (at least three slices of 32; the
    row offsets of a tile within 32 bits).
    """
    return isinstance(w, torch.Tensor) and w.is_cuda and w.dim() == 2 and w.dtype == torch.bfloat16 and \
        w.shape[0] % 16 == 0 and w.shape[1] % 32 == 0 and 96 <= w.shape[1] <= (1 << 22)


def pack_weight(w: torch.Tensor) -> PackedWeight:
    """The matrix in the blocked layout of ``PackedWeight`` (a copy; the row-major tensor can be dropped)."""
    if not packable(w):
        raise InvalidArgument(f"pack_weight takes a bfloat16 GPU matrix [N % 16 == 0, K % 32 == 0, K >= 96], got "
                              f"{list(w.shape)} {w.dtype}")
    N, K = w.shape
    blocks = w.view(N // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(N, K)
    return PackedWeight(blocks, (N, K))


def _bf16_product_operands(x, w, out, gated, what):
    _gpu(x, "matmul input")
    _gpu(w.blocks if isinstance(w, PackedWeight) else w, "matmul weight")
    _gpu(out, "matmul output")
    M, K = x.shape
    N, K2 = w.shape
    width = N // 2 if gated else N
    if K != K2 or tuple(out.shape) != (M, width):
        raise InvalidArgument(f"matmul: input {list(x.shape)}, weight {list(w.shape)}, output {list(out.shape)}")
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise InvalidArgument(f"{what} takes bfloat16 operands")
    if K % 8:
        raise InvalidArgument(f"{what} takes K % 8 == 0, got K={K}")
    if gated and (N % 16 or out.dtype != torch.bfloat16):
        raise InvalidArgument(f"{what}: a gated product needs N % 16 == 0 and a bfloat16 output")
    return M, N, K


def skinny_splits(N: int, K: int) -> int:
    """Ranges of K a decode-time product of up to 16 rows over a ``[N, K]`` weight is best cut into when its caller
    adds partial sums."""
    return int(_lib("skinny_gemm_bf16").tie_skinny_gemm_splits(N, K))


@functools.lru_cache(maxsize=None)
def few_rows_plan(M: int, N: int, K: int, gated: bool = False) -> tuple:
    """``(shares_x, tiles, splits)`` of the decode product for ``M`` rows over a packed ``[N, K]`` weight: whether the
    kernel that shares x through LDS runs (17 to 64 rows), the weight tiles a workgroup takes, and the ranges of K
    the product is best cut into when its caller adds partial sums (up to 16 rows: ``skinny_splits``)."""
    shares_x, tiles = ctypes.c_int(0), ctypes.c_int(0)
    splits = int(_lib("skinny_gemm_bf16").tie_skinny_few_rows_plan(M, N, K, int(gated), ctypes.addressof(shares_x),
                                                                  ctypes.addressof(tiles)))
    return bool(shares_x.value), tiles.value, splits


NORM_EPILOGUE_ROWS = 16      # rows up to which the decode product's epilogue does the norms' work (SkNorm)
# Whether steps of up to that many rows leave the RMS norms between their sub-layers to the products' epilogues
# (parts.Linear.prepares_norms). False: every norm is a kernel of its own (tests compare the two ways).
NORMS_IN_PRODUCTS = True


class RowScale:
    """Rows that are a norm's input times its weight, the ``1 / rms`` still to come: ``squares[m]`` holds, per
    16-column tile of the row the norm saw, the sum of its squares; the factor is
    ``1 / sqrt(squares[m].sum() / n + eps)`` and belongs on whatever product is formed from the rows."""

    __slots__ = ("squares", "n", "eps")

    def __init__(self, squares: torch.Tensor, n: int, eps: float):
        self.squares, self.n, self.eps = squares, int(n), float(eps)


def skinny_gemm_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False,
                     gated: bool = False, splits: int = 1, row_scale: Optional[RowScale] = None,
                     next_norm: Optional[tuple] = None, tiles: int = 0, loads: int = 0, waves: int = 0) -> None:
    """out (+)= x @ w.T for at most 64 rows of bfloat16 x against bfloat16 w, on the matrix cores.

    ``gated``: w is a gate/up pair interleaved by ``interleave_gate_up`` and out receives silu(gate) * up.
    ``splits`` > 1: out is ``[splits, M, N]`` float32 and receives one plane of partial sums per range
    of K, for the consumer to add (``add_partials``, or a kernel that takes planes).
    Up to ``NORM_EPILOGUE_ROWS`` rows the epilogue can do the work of the RMS norms around the product:
    ``row_scale``: x lacks its norm's ``1 / rms``, and the sums are multiplied by it (before the activation of
    a gated product); ``next_norm = (weight [N], next_x bfloat16 [M, N], squares float32 [M, N / 16])`` with
    ``accumulate`` and one plane: out is the residual stream, and beside ``out += x @ w.T`` the epilogue leaves
    ``next_x = bfloat16(out * weight)`` and the sums of ``out ** 2`` per 16-column tile for the norm that follows
    (a ``RowScale`` for whoever multiplies ``next_x``).
    """
    if splits > 1:
        if out.dim() != 3 or out.shape[0] != splits or out.dtype != torch.float32 or accumulate or gated:
            raise InvalidArgument(f"skinny_gemm_bf16: {splits} splits need a float32 output of {splits} planes, "
                                  f"got {list(out.shape)} {out.dtype}, and neither accumulate nor gated")
        M, N, K = _bf16_product_operands(x, w, out[0], gated, "skinny_gemm_bf16")
    else:
        M, N, K = _bf16_product_operands(x, w, out, gated, "skinny_gemm_bf16")
    if M > 64:
        raise InvalidArgument(f"skinny_gemm_bf16 takes at most 64 rows, got {M}")
    if gated and accumulate:
        raise InvalidArgument("a gated product does not accumulate")
    if row_scale is None and next_norm is None:
        _call(_lib("skinny_gemm_bf16").tie_skinny_gemm_bf16, "skinny_gemm_bf16",
            x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out, "matmul output"), int(accumulate), int(gated), M, N, K,
            int(splits), int(isinstance(w, PackedWeight)), _stream())
        return
    if M > NORM_EPILOGUE_ROWS:
        raise InvalidArgument(f"the product's epilogue does the norms' work for up to {NORM_EPILOGUE_ROWS} rows, not {M}")
    squares_in, tiles_in, n_in, eps_in = None, 0, 1.0, 0.0
    if row_scale is not None:
        _f32(row_scale.squares, "sums of squares")
        if row_scale.squares.dim() != 2 or row_scale.squares.shape[0] < M or not row_scale.squares.is_contiguous() \
                or row_scale.n <= 0:
            raise InvalidArgument(f"sums of squares {list(row_scale.squares.shape)} do not cover {M} rows")
        squares_in, tiles_in, n_in, eps_in = row_scale.squares, row_scale.squares.shape[1], float(row_scale.n), row_scale.eps
    next_w = next_x = squares_out = None
    if next_norm is not None:
        next_w, next_x, squares_out = next_norm
        _f32(next_w, "the next norm's weight", (N,))
        _f32(squares_out, "sums of squares", (M, N // 16))
        _gpu(next_x, "the next norm's rows")
        if splits != 1 or gated or not accumulate or out.dtype != torch.float32 or N % 16 or \
                next_x.dtype != torch.bfloat16 or tuple(next_x.shape) != (M, N) or not next_x.is_contiguous() or \
                not squares_out.is_contiguous():
            raise InvalidArgument("a product that prepares the next norm adds to a float32 stream in one plane, is not "
                                  f"gated, and leaves bfloat16 rows [{M}, {N}] (N in steps of 16)")
    _call(_lib("skinny_gemm_bf16").tie_skinny_gemm_bf16_norm, "skinny_gemm_bf16_norm",
        x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out, "matmul output"), int(accumulate), int(gated), M, N, K,
        int(splits), int(isinstance(w, PackedWeight)), _ptr(squares_in), tiles_in, n_in, eps_in, _ptr(next_w),
        _ptr(next_x), _ptr(squares_out), int(tiles), int(loads), int(waves), _stream())


def gemm_splits(M: int, N: int, K: int, packed: bool = False) -> int:
    """Ranges of K a product of M > 64 rows over a ``[N, K]`` weight is best cut into when its caller adds partial sums."""
    return int(_lib("gemm_bf16").tie_gemm_bf16_splits(M, N, K, int(packed)))


def gemm_tile(M: int, N: int, K: int, packed: bool = False, splits: int = 0) -> int:
    """The tile (``gemm_bf16``'s numbering) a product left to choose runs on, with ``splits`` ranges of K fixed (0: the plan's own)."""
    return int(_lib("gemm_bf16").tie_gemm_bf16_tile(M, N, K, int(packed), splits))


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False, tile: int = 0,
              gated: bool = False, splits: int = 1) -> None:
    """out (+)= x @ w.T for bfloat16 operands on the matrix cores, any number of rows; K % 8 == 0.

    ``tile`` picks the workgroup tile (1 = 128x128, 2 = 256x256, 3 = 256x128; 4 = 256x256, 5 = 256x128, 6 = 128x256,
    7 = 128x128, 8 = 64x256, 9 = 64x128 and 10 = 256x192 with operand slices loaded straight into LDS, which need
    K % 32 == 0 and N % 4 == 0; 0 lets the kernel choose);
    ``gated`` and ``splits`` as in ``skinny_gemm_bf16`` (planes of partial sums, ``[splits, M, N]`` float32).
    """
    if splits > 1:
        if out.dim() != 3 or out.shape[0] != splits or out.dtype != torch.float32 or accumulate or gated:
            raise InvalidArgument(f"gemm_bf16: {splits} splits need a float32 output of {splits} planes, got "
                                  f"{list(out.shape)} {out.dtype}, and neither accumulate nor gated")
        M, N, K = _bf16_product_operands(x, w, out[0], gated, "gemm_bf16")
    else:
        M, N, K = _bf16_product_operands(x, w, out, gated, "gemm_bf16")
    if accumulate and (gated or out.dtype != torch.float32):
        raise InvalidArgument("gemm_bf16 accumulates into float32 outputs only, and not in a gated product")
    _call(_lib("gemm_bf16").tie_gemm_bf16, "gemm_bf16", x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out, "matmul output"),
                                           int(accumulate), int(gated), M, N, K, tile, int(splits),
                                           int(isinstance(w, PackedWeight)), _stream())


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """The weight layout of a gated product: blocks of 16 rows = 8 gate rows then the 8 up rows of the same outputs."""
    I, K = gate.shape
    if up.shape != gate.shape or I % 8:
        raise InvalidArgument(f"gate {list(gate.shape)} and up {list(up.shape)} must match, with a multiple of 8 rows")
    return torch.stack([gate.reshape(I // 8, 8, K), up.reshape(I // 8, 8, K)], dim=1).reshape(2 * I, K).contiguous()


_few_rows_memo: Dict[tuple, bool] = {}


def decode_product_rows(M: int, w, gated: bool = False) -> bool:
    """Whether ``M`` rows against ``w`` go to the decode product (``skinny_gemm_bf16``) rather than the tiled one.

    Up to 32 rows always, above 64 never; between, the tiled product with 64-row tiles where it takes the weight
    (packed, whole slices of K), except for gated products that are not very wide (measured).
    """
    if M <= 32 or M > 64:
        return M <= 32
    N, K = w.shape
    packed = isinstance(w, PackedWeight)
    key = (M, N, K, packed, bool(gated))
    tiled = _few_rows_memo.get(key)
    if tiled is None:
        tiled = _few_rows_memo[key] = bool(_lib("gemm_bf16").tie_gemm_bf16_wins_few_rows(M, N, K, int(packed), int(gated)))
    return not tiled


def linear_swiglu(x: torch.Tensor, w_interleaved: torch.Tensor, out: torch.Tensor,
                  row_scale: Optional[RowScale] = None) -> None:
    """out = silu(x @ gate.T) * (x @ up.T) in one product over the interleaved weight; bfloat16 only.
    ``row_scale`` as in ``skinny_gemm_bf16`` (up to ``NORM_EPILOGUE_ROWS`` rows)."""
    if decode_product_rows(x.shape[0], w_interleaved, gated=True):
        skinny_gemm_bf16(x, w_interleaved, out, gated=True, row_scale=row_scale)
    elif row_scale is not None:
        raise InvalidArgument(f"{x.shape[0]} rows without their norm's factor: only the decode product applies it")
    else:
        gemm_bf16(x, w_interleaved, out, gated=True)


@functools.lru_cache(maxsize=None)
def norm_epilogue_rows(N: int, K: int) -> int:
    """The most rows for which a product over a packed ``[N, K]`` weight that ends a sub-layer is worth running
    with the next norm's work in its epilogue (``skinny_gemm_bf16(next_norm=...)``) rather than as planes that a
    norm kernel adds; 0 where it never is. Never above ``NORM_EPILOGUE_ROWS``."""
    return min(NORM_EPILOGUE_ROWS, int(_lib("skinny_gemm_bf16").tie_skinny_norm_epilogue_rows(N, K)))


def applies_row_scale(x: torch.Tensor, w) -> bool:
    """Whether ``linear`` / ``linear_swiglu`` over these operands run on the product whose epilogue applies a
    ``RowScale`` (the decode product, up to ``NORM_EPILOGUE_ROWS`` rows)."""
    # the kernel holds the tiles' sums of squares of all rows in 32 KB of LDS, 64 tiles (256 bytes) a load
    staged = x.shape[0] * (-(-(x.shape[1] // 16) // 64)) * 256
    return x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.shape[1] % 16 == 0 and \
        x.shape[0] <= NORM_EPILOGUE_ROWS and staged <= 32768


def linear(x: torch.Tensor, w, out: torch.Tensor, accumulate: bool = False, row_scale: Optional[RowScale] = None) -> None:
    """out (+)= x @ w.T, on the fastest kernel that takes these operands (w a matrix or a ``PackedWeight``).
    ``row_scale``: see ``skinny_gemm_bf16``; only where ``applies_row_scale`` says so."""
    if row_scale is not None and not (applies_row_scale(x, w) and not (accumulate and out.dtype != torch.float32)):
        raise InvalidArgument("these operands do not run on the product that applies a row scale: scale the rows first")
    if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.shape[1] % 8 == 0 and \
            not (accumulate and out.dtype != torch.float32):
        if decode_product_rows(x.shape[0], w):
            skinny_gemm_bf16(x, w, out, accumulate, row_scale=row_scale)
        else:
            gemm_bf16(x, w, out, accumulate)
    elif isinstance(w, PackedWeight):
        raise InvalidArgument(f"a packed weight is read by the bfloat16 products only: input {x.dtype}, output "
                              f"{out.dtype}, accumulate={accumulate}")
    else:
        gemm_generic(x, w, out, accumulate)


def rope_angles(positions: torch.Tensor, inv_freq: torch.Tensor, out: torch.Tensor) -> None:
    """out[t] = [cos(float(positions[t]) * inv_freq), sin(...)]: the rotation table of one step, ``[T, 2 * half]`` float32."""
    T = positions.numel()
    half = inv_freq.numel()
    _i32(positions, "positions", T)
    _f32(inv_freq, "inv_freq", (half,))
    _f32(out, "rope angles", (T, 2 * half))
    _call(_lib("elementwise").tie_rope_angles, "rope_angles", positions.data_ptr(), inv_freq.data_ptr(), out.data_ptr(), T, half,
                                               _stream())


def qk_norm_rope_kv_write(qkv: torch.Tensor, q_out: torch.Tensor, q_weight: Optional[torch.Tensor],
                          k_weight: Optional[torch.Tensor], eps: float, inv_freq: Optional[torch.Tensor],
                          positions: torch.Tensor, slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                          v_cache: Optional[torch.Tensor], num_heads: int, num_kv_heads: int, head_dim: int,
                          block_size: int, write_kv: bool = True, k_dense: Optional[torch.Tensor] = None,
                          planes: int = 1, plane_stride: int = 0, angles: Optional[torch.Tensor] = None,
                          rotary_dim: Optional[int] = None, pairing: str = "rotate_half") -> None:
    """Per-head RMSNorm of q and k, rotation by position, q to ``q_out``, k and v into the paged cache.

    The first ``rotary_dim`` dimensions of a head (default: all) are rotated, as pairs
    ``(i, i + rotary_dim / 2)`` (``pairing`` "rotate_half") or ``(2 i, 2 i + 1)`` ("interleaved") by
    ``position * inv_freq[i]``; ``inv_freq`` holds ``rotary_dim / 2`` values.

    ``angles`` (from ``rope_angles`` for the same positions and ``inv_freq``) spares the kernel the
    sines and cosines.

    With ``planes`` > 1, ``qkv`` is the first of that many planes of partial sums, ``plane_stride``
    elements apart, which are added as they are read.

    ``qkv`` is ``[T, >= (H + 2 KVH) * Dh]`` (rows may be wider than what is read). ``q_out`` is a
    ``[T, H * Dh]`` tensor or a view into ``qkv`` itself (rows ``qkv.stride(0)`` apart). With
    ``k_dense`` (``[T, KVH * Dh]`` or a view into ``qkv``) the keys go there instead of the cache
    and ``write_kv`` must be off. Null weights or ``inv_freq`` skip the norm or the rotation.
    """
    _gpu_strided(qkv, "qkv")
    _gpu_strided(q_out, "q output")
    T, in_width = qkv.shape
    in_row = qkv.stride(0)
    H, KVH, Dh = num_heads, num_kv_heads, head_dim
    heads = H + (KVH if (write_kv or k_dense is not None) else 0) + (KVH if write_kv else 0)
    if in_width < heads * Dh:
        raise InvalidArgument(f"qkv rows hold {in_width} values, {heads * Dh} are needed")
    if tuple(q_out.shape) != (T, H * Dh):
        raise InvalidArgument(f"q output has shape {list(q_out.shape)}, expected {[T, H * Dh]}")
    if Dh % 2 or Dh > MAX_HEAD_DIM:
        raise InvalidArgument(f"head_dim {Dh} must be even and at most {MAX_HEAD_DIM}")
    if T > MAX_STEP_TOKENS:
        raise InvalidArgument(f"a step of {T} tokens exceeds the {MAX_STEP_TOKENS} this kernel takes")
    for wt, nm in ((q_weight, "q_norm weight"), (k_weight, "k_norm weight")):
        if wt is not None:
            _f32(wt, nm, (Dh,))
    rotary_dim = Dh if rotary_dim is None else int(rotary_dim)
    if rotary_dim % 2 or not 0 <= rotary_dim <= Dh:
        raise InvalidArgument(f"rotary_dim {rotary_dim} must be even and at most head_dim {Dh}")
    if pairing not in ("rotate_half", "interleaved"):
        raise InvalidArgument(f"the fused kernel rotates pairs as 'rotate_half' or 'interleaved', not '{pairing}'")
    if inv_freq is not None:
        _f32(inv_freq, "inv_freq", (rotary_dim // 2,))
    if angles is not None:
        _f32(angles, "rope angles", (T, rotary_dim))
    _i32(positions, "positions", T)
    cache_code = _code(q_out, "q output")
    k_row = 0
    if k_dense is not None:
        if write_kv:
            raise InvalidArgument("keys go either to k_dense or into the cache, not both")
        _gpu_strided(k_dense, "k output")
        if tuple(k_dense.shape) != (T, KVH * Dh) or k_dense.dtype != q_out.dtype:
            raise InvalidArgument(f"k output {list(k_dense.shape)} {k_dense.dtype} does not fit {[T, KVH * Dh]}")
        k_row = k_dense.stride(0)
    if write_kv:
        _i32(slots, "slot mapping", T)
        _gpu(k_cache, "k cache")
        _gpu(v_cache, "v cache")
        _check_cache(k_cache, v_cache, KVH, block_size, Dh)
        cache_code = _cache_code(k_cache, q_out, "k cache")
    _call(_lib("elementwise").tie_qk_norm_rope_kv_write, "qk_norm_rope_kv_write",
        qkv.data_ptr(), _code(qkv, "qkv"), q_out.data_ptr(), _code(q_out, "q output"), _ptr(q_weight),
        _ptr(k_weight), float(eps), _ptr(inv_freq), _ptr(angles), positions.data_ptr(),
        _ptr(slots) if write_kv else None,
        _ptr(k_cache) if write_kv else None, _ptr(v_cache) if write_kv else None, cache_code, int(write_kv),
        _ptr(k_dense), T, H, KVH, Dh, block_size, in_row, q_out.stride(0), k_row, int(plane_stride), int(planes),
        rotary_dim, int(pairing == "interleaved"), _stream())


def paged_attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                            query_start: torch.Tensor, context_lens: torch.Tensor, block_tables: torch.Tensor,
                            seq_of_row: torch.Tensor, num_heads: int, scale: float,
                            window: Optional[int] = None) -> None:
    """Causal attention of every query row over its sequence's cached keys (float32 arithmetic, any sizes)."""
    _gpu(q, "queries")
    _gpu(out, "attention output")
    _gpu(k_cache, "k cache")
    _gpu(v_cache, "v cache")
    NB, KVH, bs, Dh = k_cache.shape
    _check_cache(k_cache, v_cache, KVH, bs, Dh)
    T = q.shape[0]
    H = num_heads
    if tuple(q.shape) != (T, H * Dh) or tuple(out.shape) != (T, H * Dh):
        raise InvalidArgument(f"attention: q {list(q.shape)} / out {list(out.shape)} do not fit {H} heads of {Dh}")
    if H % KVH:
        raise InvalidArgument(f"{H} query heads are not a multiple of {KVH} kv heads")
    if Dh > MAX_HEAD_DIM:
        raise InvalidArgument(f"head_dim {Dh} exceeds the {MAX_HEAD_DIM} this kernel takes")
    if T > MAX_STEP_TOKENS:
        raise InvalidArgument(f"a step of {T} tokens exceeds the {MAX_STEP_TOKENS} this kernel takes")
    S = context_lens.numel()
    _i32(query_start, "query_start", S + 1)
    _i32(context_lens, "context_lens")
    _i32(seq_of_row, "seq_of_row", T)
    _i32(block_tables, "block tables")
    if block_tables.dim() != 2 or block_tables.shape[0] < S:
        raise InvalidArgument(f"block tables {list(block_tables.shape)} do not cover {S} sequences")
    _call(_lib("attention_generic").tie_paged_attention_generic, "paged_attention_generic",
        q.data_ptr(), _code(q, "queries"), k_cache.data_ptr(), v_cache.data_ptr(), _cache_code(k_cache, q, "k cache"),
        out.data_ptr(), _code(out, "attention output"), query_start.data_ptr(), context_lens.data_ptr(),
        block_tables.data_ptr(), seq_of_row.data_ptr(), T, H, KVH, Dh, bs, block_tables.shape[1], float(scale),
        int(window or 0), _stream())


_argmax_workspace = {}


def argmax_rows(logits: torch.Tensor, out: torch.Tensor, max_out: Optional[torch.Tensor] = None) -> None:
    """out[r] = lowest index of the maximum of logits[r]; -1 marks a row with a NaN. ``max_out[r]`` = that maximum."""
    _f32(logits, "logits")
    R, V = logits.shape
    _i32(out, "argmax output", R)
    if max_out is not None:
        _f32(max_out, "row maxima", (R,))
    key = str(logits.device)
    ws = _argmax_workspace.get(key)
    if ws is None or ws[0].numel() < R * 64:
        rows = max(R, 64)
        ws = _argmax_workspace[key] = (torch.empty(rows * 64, dtype=torch.float32, device=logits.device),
                                       torch.empty(rows * 64, dtype=torch.int32, device=logits.device))
    _call(_lib("elementwise").tie_argmax, "argmax", logits.data_ptr(), out.data_ptr(), _ptr(max_out), ws[0].data_ptr(),
                                          ws[1].data_ptr(), R, V, _stream())


ARGMAX_STATIC_MAX_ROWS = 1024     # TIE_ARGMAX_STATIC_MAX_ROWS of csrc/argmax_static.h


def argmax_rows_static(logits: torch.Tensor, out: torch.Tensor, max_out: Optional[torch.Tensor] = None) -> None:
    """``argmax_rows`` without any allocation: the candidates between its two stages live in a static device array.

    For callers that cannot allocate (stream capture, loops that must stay off the allocator). At most
    ``ARGMAX_STATIC_MAX_ROWS`` rows; calls that may overlap on one GPU race on the shared array.
    """
    _f32(logits, "logits")
    R, V = logits.shape
    _i32(out, "argmax output", R)
    if max_out is not None:
        _f32(max_out, "row maxima", (R,))
    if R > ARGMAX_STATIC_MAX_ROWS:
        raise InvalidArgument(f"argmax_rows_static takes at most {ARGMAX_STATIC_MAX_ROWS} rows (the size of its static "
                              f"scratch array), got {R}")
    with torch.cuda.device(logits.device):
        _call(_lib("elementwise").tie_argmax_static, "argmax_static", logits.data_ptr(), out.data_ptr(), _ptr(max_out), R, V,
                                                     _stream())


MAX_SAMPLED_VOCAB = 1 << 20      # rows the temperature sampling kernel takes (the sums of its pieces fit LDS)


def _row_selection(rows: Optional[torch.Tensor], row_max: Optional[torch.Tensor], R: int) -> int:
    count = 0
    if rows is not None:
        _i32(rows, "row numbers")
        count = rows.numel()
        if not 0 < count <= R:
            raise InvalidArgument(f"{count} row numbers for {R} rows")
    if row_max is not None:
        _f32(row_max, "row maxima", (R,))
    return count


def _uniform_numbers(uniform: torch.Tensor, other_uniform, take_other, drew_none, R: int) -> None:
    for t, name in ((uniform, "uniform numbers"), (other_uniform, "the other uniform numbers")):
        if t is None:
            continue
        _gpu(t, name)
        if t.dtype != torch.float64 or t.numel() != R:
            raise InvalidArgument(f"{name} must be float64, one per row")
    if (take_other is None) != (other_uniform is None):
        raise InvalidArgument("the other uniform numbers and the marks of the rows that take them come together")
    if take_other is not None:
        _i32(take_other, "marks of the rows that take the other number", R)
    if drew_none is not None:
        _i32(drew_none, "marks of the rows that drew nothing", R)


def sample_rows(logits: torch.Tensor, inv_temperature: torch.Tensor, uniform: torch.Tensor, out: torch.Tensor,
                rows: Optional[torch.Tensor] = None, row_max: Optional[torch.Tensor] = None,
                other_uniform: Optional[torch.Tensor] = None, take_other: Optional[torch.Tensor] = None,
                drew_none: Optional[torch.Tensor] = None) -> None:
    """Draws one token per row from softmax(logits * inv_temperature) with the given uniform numbers, walking the
    tokens in index order. ``out[r]`` is -1 for a row with a NaN and -2 for a row that is all -inf. With ``rows``
    (int32 row numbers) only those rows are drawn; the other entries of ``out`` stay as they are. With ``row_max``
    (the rows' maxima) the kernel does not look for them and leaves ``out`` of a row without a finite maximum as
    it is. ``drew_none[r]`` becomes 1 where the row took no uniform number (no finite maximum), else 0;
    where ``take_other[r]`` is not 0 the row's number is ``other_uniform[r]`` (a step queued before the one
    before it is read passes that step's ``drew_none``, and both numbers its stream may be at)."""
    _f32(logits, "logits")
    if logits.dim() != 2:
        raise InvalidArgument("logits must be [rows, vocabulary]")
    R, V = logits.shape
    if V > MAX_SAMPLED_VOCAB:
        raise InvalidArgument(f"the sampling kernel takes rows of up to {MAX_SAMPLED_VOCAB} logits, got {V}")
    _f32(inv_temperature, "inverse temperatures", (R,))
    _uniform_numbers(uniform, other_uniform, take_other, drew_none, R)
    _i32(out, "sample output", R)
    count = _row_selection(rows, row_max, R)
    _call(_lib("elementwise").tie_sample, "sample", logits.data_ptr(), _ptr(row_max), inv_temperature.data_ptr(),
          uniform.data_ptr(), _ptr(other_uniform), _ptr(take_other), _ptr(drew_none), _ptr(rows), count, out.data_ptr(),
          R, V, _stream())


MAX_FILTERED_VOCAB = 1 << 19     # rows the top-k / top-p sampling kernel takes (its integer sums fit 64 bits)


def sample_rows_filtered(logits: torch.Tensor, inv_temperature: torch.Tensor, uniform: torch.Tensor,
                         top_k: torch.Tensor, top_p: torch.Tensor, out: torch.Tensor,
                         rows: Optional[torch.Tensor] = None, row_max: Optional[torch.Tensor] = None,
                         other_uniform: Optional[torch.Tensor] = None, take_other: Optional[torch.Tensor] = None,
                         drew_none: Optional[torch.Tensor] = None) -> None:
    """Draws one token per row with top-k and top-p: ``top_k[r]`` most likely kept (0: all), then the smallest
    prefix by likelihood whose weight reaches ``top_p[r]`` of the total (1: all), one uniform number a row, which
    walks the candidates in the order of likelihood also where neither filter removes any (``sample_rows`` walks
    them in index order, as the rule is without filters).
    ``out[r]`` is -1 for a row with a NaN and -2 for a row that is all -inf. With ``rows`` (int32 row numbers)
    only those rows are drawn; the other entries of ``out`` stay as they are. ``row_max``, ``other_uniform``,
    ``take_other`` and ``drew_none`` as in ``sample_rows``."""
    _f32(logits, "logits")
    if logits.dim() != 2:
        raise InvalidArgument("logits must be [rows, vocabulary]")
    R, V = logits.shape
    if V > MAX_FILTERED_VOCAB:
        raise InvalidArgument(f"the top-k / top-p kernel takes rows of up to {MAX_FILTERED_VOCAB} logits, got {V}")
    _f32(inv_temperature, "inverse temperatures", (R,))
    _f32(top_p, "top_p", (R,))
    _i32(top_k, "top_k", R)
    _uniform_numbers(uniform, other_uniform, take_other, drew_none, R)
    _i32(out, "sample output", R)
    count = _row_selection(rows, row_max, R)
    _call(_lib("sample_filtered").tie_sample_filtered, "sample_filtered", logits.data_ptr(), _ptr(row_max),
          inv_temperature.data_ptr(), uniform.data_ptr(), _ptr(other_uniform), _ptr(take_other), _ptr(drew_none),
          top_k.data_ptr(), top_p.data_ptr(), _ptr(rows), count, out.data_ptr(), R, V, _stream())


# Up to this many workgroups of single decoded rows run in the prefill attention kernel beside a step's prompt
# portions rather than in a launch (and a merge) of the decode kernel of their own; a row costs a 32-row tile
# there, so many of them are better off in the decode kernel, which takes a group's heads as its columns.
SINGLE_ROWS_RIDE_ALONG = 128
PREFILL_MAX_CACHE_BYTES = 1 << 35      # the prefill attention kernel addresses a cache plane in 32-bit units of 8 bytes


def prefill_addressable(k_cache: torch.Tensor) -> bool:
    """Whether the prefill attention kernel can address this cache plane: under 32 GB, pages under 128 MB, under 2^24 pages."""
    pages, page_bytes = k_cache.shape[0], k_cache[0].numel() * k_cache.element_size()
    return pages * page_bytes < PREFILL_MAX_CACHE_BYTES and page_bytes < (1 << 27) and pages < (1 << 24)


def mfma_block_size(block_size: int) -> bool:
    """Block sizes the matrix-core attention kernels take: powers of two from 4 (others go to the generic kernel)."""
    return block_size >= 4 and block_size & (block_size - 1) == 0


def decode_splits(num_seqs: int, num_kv_heads: int, max_context: int, block_size: int = 16) -> int:
    """How many ways the keys of each sequence are split so that a decode step fills the GPU.

    Never more than ``MAX_KEY_SPLITS``, which is what the kernel and its merge take. With pages of 16
    positions or more the kernel keeps several tiles of keys in flight a wave, a wave is a workgroup, and the
    GPU holds 1024 of them at a time, four a compute unit. About 512 waves with shares of at least 128 keys
    measured best from batch 1 to 128 where that many waves spread evenly; where they do not (24 sequences of 8
    KV heads in 3 shares are 576 waves: two compute units in three carry two, the others three) up to twice the
    shares are tried for the count that leaves the fewest compute units waiting, each further share weighed at
    1 % for what it writes and the merge reads (batch 24 at 4096 keys: 4 shares, 73.5 against 82.8 µs a layer;
    batch 40: 3 shares, 115 against 125; batch 12: 8 shares, 42 against 48). With exactly 256 (sequence, KV head)
    pairs one wave each walks its whole sequence and nothing is merged (batch 32: 93 against 96 µs). With smaller
    pages a wave has one tile in flight and the GPU wants four times the waves.
    """
    if block_size >= 16:
        pairs = max(1, num_seqs * num_kv_heads)
        if pairs == 256:
            return 1
        by_length = max(1, max_context // 128)          # at least four 32-key tiles a share
        most = min(by_length, MAX_KEY_SPLITS)
        first = -(-512 // pairs)
        if first >= most:
            return max(1, most)
        best, best_cost = first, None
        for n in range(first, min(2 * first, most) + 1):
            waves = pairs * n
            if n > first and waves > 1024:
                break
            cost = -(-waves // 256) * 256 / waves * (1 + 0.01 * n)
            if best_cost is None or cost < best_cost:
                best, best_cost = n, cost
        return best
    by_occupancy = -(-2048 // max(1, num_seqs * num_kv_heads))     # about 2048 waves ...
    if by_occupancy > 16:
        by_occupancy = -(-by_occupancy // 2)        # ... but half as many where that still leaves many shares to merge
    by_length = max(1, max_context // 64)           # at least two 32-key tiles a share
    return max(1, min(by_occupancy, by_length, MAX_KEY_SPLITS))


# Shares of one length for all sequences (``decode_share_plan``): the grid holds at least this many a sequence.
BALANCED_SHARES_GRID = 8
# Where each sequence's own shares would be this few at most, shares of one length are taken if they halve the
# longest share; with more shares of its own a sequence's waves are short already, and only a share four times
# shorter pays (16 sequences of 8 KV heads, 100 to 4000 keys, 4 shares each: 37.7 us a layer, shares of one
# length 36.8 to 44.8; one sequence of 32 k keys beside 23 of 1 k: 176 -> 74).
BALANCED_SHARES_MAX_EQUAL = 3


def decode_share_plan(context_lens, num_kv_heads: int, plan_context: int, block_size: int = 16,
                      window: Optional[int] = None) -> "tuple":
    """``(shares, share_tiles)`` for a step of single decoded tokens over sequences of these lengths.

    ``share_tiles`` = 0: every sequence's keys go into ``shares`` equal parts of its own (``decode_splits``): the
    rule for sequences of about one length. A wave walks its share tile after tile, so the longest share sets
    the kernel's time, and with sequences of very different lengths (the longest a quarter above the mean) that
    is the longest sequence's, while the waves of the short ones are done early (32 sequences of 8 KV heads, 65 k
    keys in all: 51 us a layer with 2048 each, 79 with 100 to 4000, 87 with a quarter of them 4096 long; 2 of 4096
    beside 30 of 600: 83 for 26 k keys; one of 32 k beside 7 of 1 k: 89, as much as half of 8 of 32 k). Then all
    shares get ONE length, ``share_tiles`` tiles of 32 keys: the smallest for which the waves that have keys at all
    stay within 512 (768 above 128 (sequence, KV head) pairs, 1024 above 256). A short sequence fills one share, a long one many,
    and the rest of the grid (a power of two of shares a sequence, so that a recorded step serves while the lengths
    grow) is empty (those steps: 68, 62, 43 and 52 us; 64 sequences, 2 of them long: 94 -> 53). Taken only if the
    longest share gets half as long, a quarter where a sequence's own shares are more than three: between that
    and equal the merge and the empty shares cost what the balance gains (56 sequences, a quarter long: 94 -> 109
    us at two thirds; two of 16 k beside six of 2 k: 56 -> 57 at a third).
    """
    S = len(context_lens)
    equal = decode_splits(S, num_kv_heads, plan_context, block_size)
    if block_size < 16 or S < 2 or BALANCED_SHARES_MAX_EQUAL <= 0:
        return equal, 0
    tiles = []
    for n in context_lens:
        pos = n - 1
        first = max(0, pos - window + 1) // 32 if window else 0
        tiles.append(pos // 32 + 1 - first)
    longest = max(tiles)
    if longest * S < 1.25 * sum(tiles):
        return equal, 0
    pairs = S * num_kv_heads
    target = (512 if pairs <= 128 else 768 if pairs <= 256 else 1024) // num_kv_heads      # waves with keys, a KV head
    if target <= S:
        return equal, 0
    lo, hi = max(4, -(-longest // MAX_KEY_SPLITS)), longest      # a share of at least 128 keys, the longest within the grid
    while lo < hi:                                               # the count of waves falls as the shares grow
        mid = (lo + hi) // 2
        if sum(-(-t // mid) for t in tiles) <= target:
            hi = mid
        else:
            lo = mid + 1
    before = -(-longest // equal)
    if (2 * lo > before) if equal <= BALANCED_SHARES_MAX_EQUAL else (4 * lo >= before):
        return equal, 0
    grid = BALANCED_SHARES_GRID
    while grid * lo < longest:
        grid *= 2
    return grid, lo


def step_key_shares(step, num_seqs: int, num_kv_heads: int, plan_context: int, block_size: int) -> "tuple":
    """``(shares, share_tiles tensor or None)`` of a decode step: what the step's builder planned for this cache
    group (``key_shares`` of the group's view of the step), else the rule by the step's size alone."""
    planned = getattr(step, "key_shares", None)
    if planned is not None:
        return planned
    return decode_splits(num_seqs, num_kv_heads, plan_context, block_size), None


def check_attention_sizes(num_heads: int, num_kv_heads: int, head_dim: int) -> None:
    """Refuses, when a model is built, head geometries that no attention kernel here takes."""
    if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
        raise InvalidArgument(f"{num_heads} query heads are not a positive multiple of {num_kv_heads} kv heads")
    if head_dim <= 0 or head_dim % 2 or head_dim > MAX_HEAD_DIM:
        raise InvalidArgument(f"head_dim {head_dim} must be even and at most {MAX_HEAD_DIM}: no attention kernel of "
                              f"this engine takes it")


def attention_decode_bf16(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                          query_start: torch.Tensor, context_lens: torch.Tensor, block_tables: torch.Tensor,
                          num_seqs: int, num_heads: int, scale: float, window: Optional[int], nsplit: int,
                          part_o: Optional[torch.Tensor] = None, part_ml: Optional[torch.Tensor] = None,
                          seq_ids: Optional[torch.Tensor] = None, depth: int = 0,
                          share_tiles: Optional[torch.Tensor] = None) -> None:
    """Attention for sequences that bring one new row each (``seq_ids`` selects them; None = all).

    ``share_tiles`` (one int32 on the device, or None): the length of every share in tiles of 32 keys, for steps
    whose sequences differ much in length (``decode_share_plan``); with pages of 16 positions or more and more than
    one share.

    ``depth`` picks the kernel (0: by the library's rule; 1: page lookups per lane, any page size; 2 to 4: that
    many tiles of keys in registers, pages of 16 positions or more); all give the same bits.
    """
    _gpu(q, "queries")
    _gpu(out, "attention output")
    _gpu(k_cache, "k cache")
    _gpu(v_cache, "v cache")
    NB, KVH, bs, Dh = k_cache.shape
    _check_cache(k_cache, v_cache, KVH, bs, Dh)
    H = num_heads
    if q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise InvalidArgument("attention_decode_bf16 takes bfloat16 queries, cache and output")
    if q.shape[1] != H * Dh or out.shape != q.shape:
        raise InvalidArgument(f"attention: q {list(q.shape)} / out {list(out.shape)} do not fit {H} heads of {Dh}")
    if Dh not in MFMA_HEAD_DIMS or H % KVH or H // KVH > 16 or not mfma_block_size(bs):
        raise InvalidArgument(f"attention_decode_bf16 takes head sizes in steps of 16 up to 256, at most 16 query heads "
                              f"a KV head and block sizes 4, 8, 16, ...; got head_dim {Dh}, {H}/{KVH} heads, block {bs}")
    _i32(query_start, "query_start")
    _i32(context_lens, "context_lens")
    _i32(block_tables, "block tables")
    if seq_ids is not None:
        _i32(seq_ids, "sequence ids", num_seqs)
    if not 1 <= nsplit <= MAX_KEY_SPLITS:
        raise InvalidArgument(f"attention_decode_bf16 cuts the keys into 1 to {MAX_KEY_SPLITS} shares, got {nsplit}")
    if nsplit > 1:
        _f32(part_o, "split accumulators")
        _f32(part_ml, "split maxima and sums")
        if part_o.numel() < num_seqs * H * nsplit * Dh or part_ml.numel() < num_seqs * H * nsplit * 2:
            raise InvalidArgument("the buffers for the splits are too small")
    lib = _lib("attention_decode_bf16", Dh)
    if not 0 <= depth <= 4 or (depth > 1 and bs < 16):
        raise InvalidArgument(f"attention_decode_bf16: depth {depth} with pages of {bs} positions")
    if share_tiles is not None:
        _i32(share_tiles, "the shares' length", 1)
        if nsplit == 1 or bs < 16 or depth == 1:
            raise InvalidArgument("a length for all shares goes with more than one share and pages of 16 positions or more")
    _call(lib.tie_attention_decode_bf16_with, "attention_decode_bf16",
        q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), _ptr(part_o), _ptr(part_ml),
        query_start.data_ptr(), context_lens.data_ptr(), block_tables.data_ptr(), _ptr(seq_ids), num_seqs, H, KVH, bs,
        block_tables.shape[1], float(scale), int(window or 0), nsplit, _ptr(share_tiles), depth, _stream())


def decode_attention_prepares(batch, q_dtype: torch.dtype, k_cache: torch.Tensor, num_heads: int) -> bool:
    """Whether a step runs on the decode attention kernel that makes its own queries, newest keys and values
    from the QKV projection's planes: single decoded tokens only, bfloat16, pages of 16 positions or more,
    head sizes 32, 64, 128 or 256, at most 16 query heads a KV head, fewer than 512 (sequence, KV head) pairs."""
    NB, KVH, bs, Dh = k_cache.shape
    if not (batch.all_decode and q_dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16
            and Dh in (32, 64, 128, 256) and bs >= 16 and mfma_block_size(bs)
            and num_heads % KVH == 0 and num_heads // KVH <= 16):
        return False
    # With so many sequences that the keys are not cut into shares, every wave would make a newest key and value
    # and attend to it after its tiles, and the step is a little slower that way than with the q/k kernel before
    # it (batch 64 at the 8B shape: 0.7 %).
    return batch.num_seqs * KVH < 512


def paged_attention_prepared(planes: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                             eps: float, angles: torch.Tensor, write_kv: bool, k_cache: torch.Tensor,
                             v_cache: torch.Tensor, out: torch.Tensor, step, batch, num_heads: int, scale: float,
                             window: Optional[int], scratch) -> None:
    """Attention of a step of single decoded tokens straight from the QKV projection's planes of partial sums
    (``planes`` float32 ``[P, rows, (H + 2 KVH) * Dh]``): the kernel sums the planes, applies the per-head
    RMS norm (weights or None) and the rotation by ``angles`` (``[rows, Dh]``: cos, then sin), writes the newest
    key and value into the cache (unless ``write_kv`` is false) and attends; see ``decode_attention_prepares``."""
    NB, KVH, bs, Dh = k_cache.shape
    _check_cache(k_cache, v_cache, KVH, bs, Dh)
    H, S = num_heads, batch.num_seqs
    if not decode_attention_prepares(batch, out.dtype, k_cache, H):
        raise InvalidArgument("this step does not run on the decode attention kernel that prepares its own queries")
    _f32(planes, "QKV planes")
    _f32(angles, "rotation angles")
    _gpu(out, "attention output")
    P, rows, width = planes.shape
    if not planes.is_contiguous() or width < (H + 2 * KVH) * Dh or rows != out.shape[0] or out.shape[1] != H * Dh:
        raise InvalidArgument(f"QKV planes {list(planes.shape)} / out {list(out.shape)} do not fit {H} + 2 x {KVH} heads of {Dh}")
    if angles.shape != (rows, Dh) or not angles.is_contiguous() or not 1 <= P <= 8:
        raise InvalidArgument(f"angles {list(angles.shape)} for {rows} rows of head_dim {Dh}, {P} planes")
    for w, name in ((q_weight, "q norm weight"), (k_weight, "k norm weight")):
        if w is not None:
            _f32(w, name, (Dh,))
    nsplit, share_tiles = step_key_shares(step, S, KVH, batch.plan_context, bs)
    part_o = part_ml = None
    if nsplit > 1:
        part_o = scratch("attention.split_o", (S * H * nsplit * Dh,), torch.float32)
        part_ml = scratch("attention.split_ml", (S * H * nsplit * 2,), torch.float32)
    _call(_lib("attention_decode_bf16", Dh).tie_attention_decode_prepared_bf16, "attention_decode_prepared_bf16",
          planes.data_ptr(), rows * width, P, width, _ptr(q_weight), _ptr(k_weight), float(eps), angles.data_ptr(),
          int(bool(write_kv)), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), _ptr(part_o), _ptr(part_ml),
          batch.query_start.data_ptr(), batch.context_lens.data_ptr(), step.block_tables.data_ptr(), None, S, H, KVH,
          bs, step.block_tables.shape[1], float(scale), int(window or 0), nsplit, _ptr(share_tiles), 0, _stream())


def prefill_items(new_tokens, group_size: int) -> "list":
    """Work items ``(sequence, first new row)`` of the prefill attention kernel for one step.

    An item is one workgroup: 32, 64 or 128 consecutive new rows of a sequence, depending on how
    many query heads share a KV head (four (head, 32-row tile) pairs run side by side).
    """
    heads_at_once = min(group_size, 4)
    rows = 32 * (1 if heads_at_once >= 3 else 4 // heads_at_once)
    items = []
    for s, n in enumerate(new_tokens):
        for first in range(0, n, rows):
            items.append((s, first))
    return items


def prefill_loads_straight(head_dim: int, block_size: int) -> bool:
    """Whether the prefill attention kernel that loads its tiles straight into LDS takes this geometry
    (it has no limit on the cache's size: its addresses are 64-bit scalars)."""
    return head_dim in (32, 64, 128, 256) and block_size >= 16 and mfma_block_size(block_size)


def attention_prefill_bf16(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                           query_start: torch.Tensor, context_lens: torch.Tensor, block_tables: torch.Tensor,
                           items: torch.Tensor, num_heads: int, scale: float, window: Optional[int] = None,
                           nsplit: int = 1, part_o: Optional[torch.Tensor] = None,
                           part_ml: Optional[torch.Tensor] = None, merge_rows: Optional[torch.Tensor] = None,
                           staging: int = 0) -> None:
    """Causal attention of the new rows of the sequences ``items`` names over their cached keys.

    ``staging`` picks how key tiles reach LDS: 1 = copied through registers (any page and head size),
    2 = loaded straight into LDS (``prefill_loads_straight``), 0 = the second where it applies.

    ``nsplit`` > 1 cuts every item's keys into that many shares (one workgroup each) for steps with few
    items and long contexts; ``part_o`` / ``part_ml`` (float32, ``rows * H * nsplit * Dh`` and ``* 2``
    with rows = all rows of the step) take the partial results and ``merge_rows`` lists the rows
    that the items cover, which a second kernel then merges.
    """
    _gpu(q, "queries")
    _gpu(out, "attention output")
    _gpu(k_cache, "k cache")
    _gpu(v_cache, "v cache")
    NB, KVH, bs, Dh = k_cache.shape
    _check_cache(k_cache, v_cache, KVH, bs, Dh)
    H = num_heads
    if q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise InvalidArgument("attention_prefill_bf16 takes bfloat16 queries, cache and output")
    if q.shape[1] != H * Dh or out.shape != q.shape:
        raise InvalidArgument(f"attention: q {list(q.shape)} / out {list(out.shape)} do not fit {H} heads of {Dh}")
    if Dh not in MFMA_HEAD_DIMS or H % KVH or not mfma_block_size(bs):
        raise InvalidArgument(f"attention_prefill_bf16 takes head sizes in steps of 16 up to 256 and block sizes 4, 8, "
                              f"16, ...; got head_dim {Dh}, {H}/{KVH} heads, block {bs}")
    if staging not in (0, 1, 2) or (staging == 2 and not prefill_loads_straight(Dh, bs)):
        raise InvalidArgument(f"attention_prefill_bf16: staging {staging} with head_dim {Dh} and pages of {bs} positions")
    if staging == 0:
        staging = 2 if prefill_loads_straight(Dh, bs) else 1
    if staging == 1 and not prefill_addressable(k_cache):
        raise InvalidArgument(f"attention_prefill_bf16 addresses cache planes under 32 GB (pages under 128 MB, under 2^24 "
                              f"pages); got {NB} pages of {k_cache[0].numel() * k_cache.element_size()} bytes")
    _i32(query_start, "query_start")
    _i32(context_lens, "context_lens")
    _i32(block_tables, "block tables")
    _i32(items, "work items")
    if items.dim() != 2 or items.shape[1] != 2 or items.shape[0] == 0:
        raise InvalidArgument("work items must be a non-empty [n, 2] tensor")
    num_merge = 0
    if nsplit > 1:
        _f32(part_o, "split accumulators")
        _f32(part_ml, "split maxima and sums")
        _i32(merge_rows, "rows to merge")
        rows = q.shape[0]
        num_merge = merge_rows.numel()
        if part_o.numel() < rows * H * nsplit * Dh or part_ml.numel() < rows * H * nsplit * 2 or not 0 < num_merge <= 65535:
            raise InvalidArgument("the buffers for the splits are too small, or no (or too many) rows to merge")
    lib = _lib("attention_prefill_bf16", Dh)
    _call(lib.tie_attention_prefill_bf16_with, "attention_prefill_bf16",
        q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), query_start.data_ptr(),
        context_lens.data_ptr(), block_tables.data_ptr(), items.data_ptr(), items.shape[0], H, KVH, bs,
        block_tables.shape[1], float(scale), int(window or 0), int(nsplit), _ptr(part_o), _ptr(part_ml),
        _ptr(merge_rows), num_merge, staging, _stream())


def prefill_splits(num_items: int, num_kv_heads: int, group_size: int, max_context: int, num_rows: int) -> int:
    """Shares the keys of every prefill item are cut into: more than one only where the items alone leave CUs idle."""
    passes = -(-group_size // min(group_size, 4))
    workgroups = num_items * num_kv_heads * passes
    if workgroups >= 256 or num_rows > 65535:
        return 1
    by_fill = 512 // max(1, workgroups)
    by_length = max(1, -(-max_context // 64) // 4)          # at least four 64-key tiles a share
    return max(1, min(8, by_fill, by_length))


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor, step, batch,
                    num_heads: int, scale: float, window: Optional[int] = None, scratch=None) -> None:
    """Causal attention over the paged cache for one step's batch, on the fastest kernel that takes it.

    ``step`` is the cache group's view of the step (block tables), ``batch`` the step's arrays
    (query_start, context_lens, seq_of_row) and host-side numbers; ``scratch(name, shape, dtype)``
    hands out workspace for the partial results of split keys.
    """
    NB, KVH, bs, Dh = k_cache.shape
    fast = (q.dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16 and Dh in MFMA_HEAD_DIMS
            and num_heads % KVH == 0 and mfma_block_size(bs) and scratch is not None)
    if fast and batch.all_decode and num_heads // KVH <= 16:
        S = batch.num_seqs
        nsplit, share_tiles = step_key_shares(step, S, KVH, batch.plan_context, bs)
        part_o = part_ml = None
        if nsplit > 1:
            part_o = scratch("attention.split_o", (S * num_heads * nsplit * Dh,), torch.float32)
            part_ml = scratch("attention.split_ml", (S * num_heads * nsplit * 2,), torch.float32)
        attention_decode_bf16(q, k_cache, v_cache, out, batch.query_start, batch.context_lens, step.block_tables,
                              S, num_heads, scale, window, nsplit, part_o, part_ml, share_tiles=share_tiles)
        return
    if fast:
        # A mixed step: sequences that bring one decoded token go to the decode kernel (their keys are
        # split over many waves), the prompt portions to the prefill kernel. Built once a step.
        G = num_heads // KVH
        key = ("attention_work", G)
        work = batch.memo.get(key)
        if work is None:
            new = batch.host_new_tokens
            single = [s for s, n in enumerate(new) if n == 1] if G <= 16 else []
            if len(single) == len(new):
                single = []                                   # nothing but single rows and yet not a decode step
            elif len(single) * KVH * -(-G // min(G, 4)) <= SINGLE_ROWS_RIDE_ALONG:
                single = []         # a few single rows: items of the prefill kernel, one launch and one merge less
            taken = set(single)
            items = [it for it in prefill_items(new, G) if it[0] not in taken]
            starts = [0]
            for n in new:
                starts.append(starts[-1] + n)
            merge_rows = [starts[s] + r for s in sorted({it[0] for it in items}) for r in range(new[s])]
            work = batch.memo[key] = (
                torch.tensor(single, dtype=torch.int32).to(q.device) if single else None, len(single),
                torch.tensor(items, dtype=torch.int32).to(q.device) if items else None, len(items),
                torch.tensor(merge_rows, dtype=torch.int32).to(q.device) if items else None,
                max((batch.host_context_lens[it[0]] for it in items), default=0))
        seq_ids, num_single, items, num_items, merge_rows, items_context = work
        if num_single:
            shares_key = ("single_row_shares", KVH, window)
            planned = batch.memo.get(shares_key)
            if planned is None:                # this step runs eagerly: the shares' length goes to the device by itself
                lens = [c for c, n in zip(batch.host_context_lens, batch.host_new_tokens) if n == 1]
                nsplit, length = decode_share_plan(lens, KVH, batch.plan_context, bs, window)
                planned = batch.memo[shares_key] = (
                    nsplit, torch.tensor([length], dtype=torch.int32).to(q.device) if length else None)
            nsplit, share_tiles = planned
            part_o = part_ml = None
            if nsplit > 1:
                part_o = scratch("attention.split_o", (num_single * num_heads * nsplit * Dh,), torch.float32)
                part_ml = scratch("attention.split_ml", (num_single * num_heads * nsplit * 2,), torch.float32)
            attention_decode_bf16(q, k_cache, v_cache, out, batch.query_start, batch.context_lens, step.block_tables,
                                  num_single, num_heads, scale, window, nsplit, part_o, part_ml, seq_ids=seq_ids,
                                  share_tiles=share_tiles)
        if items is not None and not prefill_loads_straight(Dh, bs) and not prefill_addressable(k_cache):
            # A cache plane the prefill kernel cannot address: the prompt portions go to the generic kernel
            # (which runs every row of the step; the single rows above are simply computed again).
            paged_attention_generic(q, k_cache, v_cache, out, batch.query_start, batch.context_lens, step.block_tables,
                                    batch.seq_of_row, num_heads, scale, window)
            return
        if items is not None:
            rows = q.shape[0]
            # by the longest context among the portions themselves: a single row of 32 k keys beside them says nothing
            # about how many tiles a portion's share would hold
            nsplit = prefill_splits(num_items, KVH, G, items_context, rows)
            part_o = part_ml = None
            if nsplit > 1:
                part_o = scratch("attention.prefill_split_o", (rows * num_heads * nsplit * Dh,), torch.float32)
                part_ml = scratch("attention.prefill_split_ml", (rows * num_heads * nsplit * 2,), torch.float32)
            attention_prefill_bf16(q, k_cache, v_cache, out, batch.query_start, batch.context_lens,
                                   step.block_tables, items, num_heads, scale, window, nsplit, part_o, part_ml,
                                   merge_rows if nsplit > 1 else None)
        return
    paged_attention_generic(q, k_cache, v_cache, out, batch.query_start, batch.context_lens, step.block_tables,
                            batch.seq_of_row, num_heads, scale, window)
