"""The operations of the engine, each one a hand-written HIP kernel for gfx950.

Every function here checks its operands on the host (device, dtype, shape,
contiguity) and then launches the kernel on the current HIP stream. There is
no CPU path: an operand that is not on a GPU, a missing compiler or a library
that cannot be loaded raise KernelUnavailable. Sizes a kernel cannot take raise
InvalidArgument before anything is launched.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..errors import InvalidArgument, KernelUnavailable
from . import build

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}

_c_int, _c_float, _c_void = ctypes.c_int, ctypes.c_float, ctypes.c_void_p

# library key -> (file stem, source)
_SOURCES = {
    "elementwise": ("tie_elementwise", "elementwise.hip"),
    "gemm_generic": ("tie_gemm_generic", "gemm_generic.hip"),
    "attention_generic": ("tie_attention_generic", "attention_generic.hip"),
}

_SIGNATURES = {
    "elementwise": {
        "tie_embed": [_c_void, _c_int, _c_void, _c_void, _c_int, _c_int, _c_void],
        "tie_rms_norm": [_c_void, _c_int, _c_void, _c_float, _c_void, _c_int, _c_void, _c_int, _c_int, _c_void],
        "tie_swiglu": [_c_void, _c_int, _c_void, _c_int, _c_int, _c_int, _c_void],
        "tie_cast": [_c_void, _c_int, _c_void, _c_int, ctypes.c_longlong, _c_void],
        "tie_qk_norm_rope_kv_write": [_c_void, _c_int, _c_void, _c_int, _c_void, _c_void, _c_float, _c_void,
                                      _c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_void, _c_int, _c_int,
                                      _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
        "tie_argmax": [_c_void, _c_void, _c_int, _c_int, _c_void],
        "tie_sample": [_c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_void],
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
}

_libs = {}


def library_list(extra_defines=None):
    """``(name, source, defines)`` of every library, for building them all."""
    return [(stem, source, {}) for stem, source in _SOURCES.values()]


def _lib(key: str):
    lib = _libs.get(key)
    if lib is None:
        stem, source = _SOURCES[key]
        lib = build.load_library(stem, source)
        for fn, argtypes in _SIGNATURES[key].items():
            f = getattr(lib, fn)
            f.argtypes = argtypes
            f.restype = _c_int
        _libs[key] = lib
    return lib


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


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


def _code(t: torch.Tensor, name: str) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise InvalidArgument(f"{name} must be float32 or bfloat16, got {t.dtype}") from None


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
    _check(_lib("elementwise").tie_embed(table.data_ptr(), _code(table, "embedding table"), ids.data_ptr(),
                                         out.data_ptr(), T, D, _stream()), "embed")


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
    _check(_lib("elementwise").tie_rms_norm(x.data_ptr(), _code(x, "rms_norm input"), weight.data_ptr(), float(eps),
                                            out.data_ptr(), _code(out, "rms_norm output"), _ptr(rows), R, n,
                                            _stream()), "rms_norm")


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i] for gate_up of shape [T, 2I]."""
    _gpu(gate_up, "swiglu input")
    _gpu(out, "swiglu output")
    T, two_i = gate_up.shape
    if two_i % 2 or tuple(out.shape) != (T, two_i // 2):
        raise InvalidArgument(f"swiglu: input {list(gate_up.shape)} and output {list(out.shape)} do not match")
    _check(_lib("elementwise").tie_swiglu(gate_up.data_ptr(), _code(gate_up, "swiglu input"), out.data_ptr(),
                                          _code(out, "swiglu output"), T, two_i // 2, _stream()), "swiglu")


def cast(x: torch.Tensor, out: torch.Tensor) -> None:
    _gpu(x, "cast input")
    _gpu(out, "cast output")
    if x.numel() != out.numel():
        raise InvalidArgument("cast: sizes differ")
    _check(_lib("elementwise").tie_cast(x.data_ptr(), _code(x, "cast input"), out.data_ptr(),
                                        _code(out, "cast output"), x.numel(), _stream()), "cast")


def gemm_generic(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """out (+)= x @ w.T with float32 multiply-adds; operands float32 or bfloat16 in any mix."""
    _gpu(x, "matmul input")
    _gpu(w, "matmul weight")
    _gpu(out, "matmul output")
    T, K = x.shape
    N, K2 = w.shape
    if K != K2 or tuple(out.shape) != (T, N):
        raise InvalidArgument(f"matmul: input {list(x.shape)}, weight {list(w.shape)}, output {list(out.shape)}")
    _check(_lib("gemm_generic").tie_gemm_generic(
        x.data_ptr(), _code(x, "matmul input"), w.data_ptr(), _code(w, "matmul weight"), out.data_ptr(),
        _code(out, "matmul output"), int(accumulate), T, N, K, _stream()), "gemm_generic")


def linear(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """out (+)= x @ w.T, on the fastest kernel that takes these operands."""
    gemm_generic(x, w, out, accumulate)


def qk_norm_rope_kv_write(qkv: torch.Tensor, q_out: torch.Tensor, q_weight: Optional[torch.Tensor],
                          k_weight: Optional[torch.Tensor], eps: float, inv_freq: Optional[torch.Tensor],
                          positions: torch.Tensor, slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                          v_cache: Optional[torch.Tensor], num_heads: int, num_kv_heads: int, head_dim: int,
                          block_size: int, write_kv: bool = True, k_dense: Optional[torch.Tensor] = None) -> None:
    """Per-head RMSNorm of q and k, rotation by position, q to ``q_out``, k and v into the paged cache.

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
    if Dh % 2 or Dh > 512:
        raise InvalidArgument(f"head_dim {Dh} must be even and at most 512")
    if T > 65535:
        raise InvalidArgument(f"a step of {T} tokens exceeds the 65535 this kernel takes")
    for wt, nm in ((q_weight, "q_norm weight"), (k_weight, "k_norm weight")):
        if wt is not None:
            _f32(wt, nm, (Dh,))
    if inv_freq is not None:
        _f32(inv_freq, "inv_freq", (Dh // 2,))
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
        if k_cache.shape != v_cache.shape or k_cache.dtype != v_cache.dtype or k_cache.dim() != 4 or \
                k_cache.shape[1] != KVH or k_cache.shape[2] != block_size or k_cache.shape[3] != Dh:
            raise InvalidArgument(f"KV cache planes {list(k_cache.shape)} / {list(v_cache.shape)} do not fit "
                                  f"{KVH} kv heads, block size {block_size}, head_dim {Dh}")
        cache_code = _code(k_cache, "k cache")
    _check(_lib("elementwise").tie_qk_norm_rope_kv_write(
        qkv.data_ptr(), _code(qkv, "qkv"), q_out.data_ptr(), _code(q_out, "q output"), _ptr(q_weight),
        _ptr(k_weight), float(eps), _ptr(inv_freq), positions.data_ptr(), _ptr(slots) if write_kv else None,
        _ptr(k_cache) if write_kv else None, _ptr(v_cache) if write_kv else None, cache_code, int(write_kv),
        _ptr(k_dense), T, H, KVH, Dh, block_size, in_row, q_out.stride(0), k_row, _stream()),
        "qk_norm_rope_kv_write")


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
    T = q.shape[0]
    H = num_heads
    if tuple(q.shape) != (T, H * Dh) or tuple(out.shape) != (T, H * Dh):
        raise InvalidArgument(f"attention: q {list(q.shape)} / out {list(out.shape)} do not fit {H} heads of {Dh}")
    if H % KVH:
        raise InvalidArgument(f"{H} query heads are not a multiple of {KVH} kv heads")
    if Dh > 512:
        raise InvalidArgument(f"head_dim {Dh} exceeds the 512 this kernel takes")
    if T > 65535:
        raise InvalidArgument(f"a step of {T} tokens exceeds the 65535 this kernel takes")
    S = context_lens.numel()
    _i32(query_start, "query_start", S + 1)
    _i32(context_lens, "context_lens")
    _i32(seq_of_row, "seq_of_row", T)
    _i32(block_tables, "block tables")
    if block_tables.dim() != 2 or block_tables.shape[0] < S:
        raise InvalidArgument(f"block tables {list(block_tables.shape)} do not cover {S} sequences")
    _check(_lib("attention_generic").tie_paged_attention_generic(
        q.data_ptr(), _code(q, "queries"), k_cache.data_ptr(), v_cache.data_ptr(), _code(k_cache, "k cache"),
        out.data_ptr(), _code(out, "attention output"), query_start.data_ptr(), context_lens.data_ptr(),
        block_tables.data_ptr(), seq_of_row.data_ptr(), T, H, KVH, Dh, bs, block_tables.shape[1], float(scale),
        int(window or 0), _stream()), "paged_attention_generic")


def argmax_rows(logits: torch.Tensor, out: torch.Tensor) -> None:
    """out[r] = lowest index of the maximum of logits[r]; -1 marks a row with a NaN."""
    _f32(logits, "logits")
    R, V = logits.shape
    _i32(out, "argmax output", R)
    _check(_lib("elementwise").tie_argmax(logits.data_ptr(), out.data_ptr(), R, V, _stream()), "argmax")


def sample_rows(logits: torch.Tensor, inv_temperature: torch.Tensor, uniform: torch.Tensor,
                out: torch.Tensor) -> None:
    """Draws one token per row from softmax(logits * inv_temperature) with the given uniform numbers."""
    _f32(logits, "logits")
    R, V = logits.shape
    _f32(inv_temperature, "inverse temperatures", (R,))
    _gpu(uniform, "uniform numbers")
    if uniform.dtype != torch.float64 or uniform.numel() != R:
        raise InvalidArgument("uniform numbers must be float64, one per row")
    _i32(out, "sample output", R)
    _check(_lib("elementwise").tie_sample(logits.data_ptr(), inv_temperature.data_ptr(), uniform.data_ptr(),
                                          out.data_ptr(), R, V, _stream()), "sample")


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor, step, batch,
                    num_heads: int, scale: float, window: Optional[int] = None) -> None:
    """Causal attention over the paged cache for one step's batch, on the fastest kernel that takes it.

    ``step`` is the cache group's view of the step (block tables), ``batch`` the step's arrays
    (query_start, context_lens, seq_of_row).
    """
    paged_attention_generic(q, k_cache, v_cache, out, batch.query_start, batch.context_lens, step.block_tables,
                            batch.seq_of_row, num_heads, scale, window)
