"""Loader and thin wrappers of the C-ABI library (libnatten_amd.so).

Counterpart of the reference's op boundary, src/natten/_libnatten/__init__.py:26-113 and
src/natten/_libnatten/torch_wrappers.py:657-716, :1373-1503: outputs are allocated here with
torch and written by the native code on torch's current stream.  There is no fallback: when
the library is missing every op raises ImportError (the reference's stubs do the same,
src/natten/_libnatten/stubs.py:25-31).
"""

from __future__ import annotations

import contextlib
import ctypes
import functools
import os
from typing import Optional, Sequence, Tuple

import torch
from torch import Tensor

_HERE = os.path.dirname(os.path.abspath(__file__))
# NATTEN_AMD_LIBRARY: another build of the library (the timing-only ones of natten_amd.build --ablate)
LIB_PATH = os.environ.get("NATTEN_AMD_LIBRARY") or os.path.join(_HERE, "libnatten_amd.so")

ABI_VERSION = 16

DTYPE_CODES = {
    torch.float16: 0,
    torch.bfloat16: 1,
    torch.float8_e4m3fn: 2,
    torch.float32: 3,
    torch.float8_e5m2: 4,
}
FP8_DTYPES = (torch.float8_e4m3fn, torch.float8_e5m2)

_lib = None
_load_error: Optional[str] = None

_SIGNATURES = {
    "natten_amd_abi_version": (ctypes.c_int, []),
    "natten_amd_last_error": (ctypes.c_char_p, []),
    "natten_amd_window": (ctypes.c_int, [ctypes.c_int] * 5 + [ctypes.c_void_p] * 2),
    "natten_amd_tile_key_mask": (ctypes.c_int, [ctypes.c_void_p] * 4),
    "natten_amd_fna_fully_block_sparse": (ctypes.c_int, [ctypes.c_int] + [ctypes.c_void_p] * 7 + [ctypes.c_int, ctypes.c_void_p]),
    "natten_amd_fna_wave_box": (ctypes.c_int, [ctypes.c_int] + [ctypes.c_void_p] * 7 + [ctypes.c_int, ctypes.c_void_p]),
    "natten_amd_fna_supported_tiles": (
        ctypes.c_int,
        [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int],
    ),
    "natten_amd_fna_forward": (
        ctypes.c_int,
        [ctypes.c_void_p] * 5
        + [ctypes.c_int] * 8
        + [ctypes.c_void_p] * 9
        + [ctypes.c_float]
        + [ctypes.c_void_p] * 3
        + [ctypes.c_int, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p],
    ),
    "natten_amd_fna_forward_workspace_bytes": (ctypes.c_uint64, []),
    "natten_amd_fna_forward_fused": (
        ctypes.c_int,
        [ctypes.c_void_p] * 5 + [ctypes.c_int] * 6 + [ctypes.c_void_p] * 7 + [ctypes.c_float] + [ctypes.c_void_p] * 3
        + [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p],
    ),
    "natten_amd_fna_forward_fused_split": (
        ctypes.c_int,
        [ctypes.c_void_p] * 5 + [ctypes.c_int] * 6 + [ctypes.c_void_p] * 7 + [ctypes.c_float]
        + [ctypes.c_int, ctypes.c_int, ctypes.c_void_p],
    ),
    "natten_amd_fna_forward_fused_static": (
        ctypes.c_int,
        [ctypes.c_void_p] * 5 + [ctypes.c_int] * 6 + [ctypes.c_void_p] * 7 + [ctypes.c_float] + [ctypes.c_void_p] * 4,
    ),
    "natten_amd_attention_forward": (
        ctypes.c_int,
        [ctypes.c_void_p] * 5 + [ctypes.c_int] * 8 + [ctypes.c_float] + [ctypes.c_void_p] * 4,
    ),
    "natten_amd_attention_forward_varlen": (
        ctypes.c_int,
        [ctypes.c_void_p] * 5 + [ctypes.c_int] * 9 + [ctypes.c_void_p] * 2 + [ctypes.c_int, ctypes.c_float]
        + [ctypes.c_void_p] * 4,
    ),
    "natten_amd_query_range": (ctypes.c_int, [ctypes.c_int] * 7 + [ctypes.c_void_p] * 2),
    "natten_amd_compute_delta": (
        ctypes.c_int,
        [ctypes.c_void_p] * 3 + [ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p],
    ),
    "natten_amd_fna_backward": (
        ctypes.c_int,
        [ctypes.c_void_p] * 10 + [ctypes.c_int] * 8 + [ctypes.c_void_p] * 9 + [ctypes.c_float, ctypes.c_void_p],
    ),
    "natten_amd_fna_backward_fused": (
        ctypes.c_int,
        [ctypes.c_void_p] * 10 + [ctypes.c_int] * 6 + [ctypes.c_void_p] * 7
        + [ctypes.c_float, ctypes.c_int, ctypes.c_void_p],
    ),
    "natten_amd_attention_backward": (
        ctypes.c_int,
        [ctypes.c_void_p] * 10 + [ctypes.c_int] * 10 + [ctypes.c_float, ctypes.c_void_p],
    ),
    "natten_amd_attention_backward_varlen": (
        ctypes.c_int,
        [ctypes.c_void_p] * 10 + [ctypes.c_int] * 4 + [ctypes.c_void_p] * 4 + [ctypes.c_int] * 6
        + [ctypes.c_float, ctypes.c_void_p],
    ),
    "natten_amd_token_permute_widen": (
        ctypes.c_int,
        [ctypes.c_void_p] * 2 + [ctypes.c_int] * 5 + [ctypes.c_void_p] * 3 + [ctypes.c_int, ctypes.c_void_p],
    ),
    "natten_amd_mfma_probe": (
        ctypes.c_int,
        [ctypes.c_void_p] * 3 + [ctypes.c_int] * 2 + [ctypes.c_void_p],
    ),
    "natten_amd_token_permute": (
        ctypes.c_int,
        [ctypes.c_void_p] * 2 + [ctypes.c_int] * 5 + [ctypes.c_void_p] * 3 + [ctypes.c_int, ctypes.c_void_p],
    ),
    "natten_amd_token_unpermute": (
        ctypes.c_int,
        [ctypes.c_void_p] * 2 + [ctypes.c_int] * 5 + [ctypes.c_void_p] * 3 + [ctypes.c_int, ctypes.c_void_p],
    ),
    "natten_amd_merge_attentions": (
        ctypes.c_int,
        [ctypes.c_void_p] * 6 + [ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p],
    ),
    "natten_amd_merge_attention_parts": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int64,
         ctypes.c_int, ctypes.c_void_p],
    ),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def _try_load():
    global _lib, _load_error
    if _lib is not None or _load_error is not None:
        return
    if not os.path.exists(LIB_PATH):
        _load_error = (
            f"natten_amd: native library not found at {LIB_PATH}. Build it with "
            "`python -m natten_amd.build` (hipcc, --offload-arch=gfx950)."
        )
        return
    try:
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.natten_amd_abi_version() != ABI_VERSION:
            raise OSError(f"ABI version {lib.natten_amd_abi_version()} != expected {ABI_VERSION}")
        _lib = lib
    except (OSError, AttributeError) as e:  # pragma: no cover - depends on the build
        _load_error = f"natten_amd: failed to load {LIB_PATH}: {e}"


@torch.compiler.assume_constant_result
def has_lib() -> bool:
    _try_load()
    return _lib is not None


def lib():
    _try_load()
    if _lib is None:
        raise ImportError(_load_error)
    return _lib


@functools.lru_cache(maxsize=4096)
def _i32_array(values: Tuple[int, ...]):
    return (ctypes.c_int32 * len(values))(*values)


def _i32(values: Sequence[int]):
    # (the arrays are only ever read, by the library: equal tuples share one)
    return _i32_array(tuple(int(v) for v in values))


def _check(rc: int):
    if rc != 0:
        raise RuntimeError(lib().natten_amd_last_error().decode())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: Tensor) -> int:
    """Handle of torch's current stream on the tensor's device (the capturing stream under graph capture)."""
    if _raw_stream is not None and t.device.index is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


_NO_GUARD = contextlib.nullcontext()


def _on_device(t: Tensor):
    """Context that makes the tensor's device current for the launch; nothing when it already is."""
    idx = t.device.index
    if idx is None or idx == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(idx)


def _require_gpu(*tensors: Tensor):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("natten_amd native ops need tensors on the GPU device.")
        if not t.is_contiguous():
            raise RuntimeError("natten_amd native ops need contiguous tensors.")


def supported_tile_sizes(dtype: torch.dtype, head_dim: int):
    if dtype not in DTYPE_CODES:
        return []
    n = lib().natten_amd_fna_supported_tiles(DTYPE_CODES[dtype], head_dim, None, None, 0)
    if n <= 0:
        return []
    q = (ctypes.c_int32 * n)()
    kv = (ctypes.c_int32 * n)()
    lib().natten_amd_fna_supported_tiles(DTYPE_CODES[dtype], head_dim, q, kv, n)
    return [(int(a), int(b)) for a, b in zip(q, kv)]


def _scale_ptrs(q: Tensor, k: Tensor, q_scale, k_scale, v_scale):
    """Device pointers (or None) of the per-head scale arrays, after checking shape/dtype/device."""
    ptrs = []
    for name, s, heads in (("q_scale", q_scale, q.shape[-2]), ("k_scale", k_scale, k.shape[-2]), ("v_scale", v_scale, k.shape[-2])):
        if s is None:
            ptrs.append(None)
            continue
        if s.dtype != torch.float32 or s.device != q.device or not s.is_contiguous() or tuple(s.shape) != (heads,):
            raise ValueError(f"{name} must be a contiguous float32 tensor of shape ({heads},) on {q.device}.")
        ptrs.append(s.data_ptr())
    return ptrs


def fna_forward(
    q: Tensor, k: Tensor, v: Tensor,
    kernel_size, stride, dilation, is_causal, scale: float,
    q_shape, kv_shape, qkv_shape, q_tile_shape, kv_tile_shape,
    q_scale: Optional[Tensor] = None, k_scale: Optional[Tensor] = None, v_scale: Optional[Tensor] = None,
    run_persistent: bool = False,
) -> Tuple[Tensor, Tensor]:
    """Token-permuted q [B*G, SQ, H, D], k/v [B*G, SK, Hkv, D] -> (out, lse float32 [B*G, SQ, H]).

    q_scale [H], k_scale / v_scale [Hkv]: optional float32 per-head dequantisation scales.
    run_persistent: work-queue launch (as many workgroups as stay resident pull Q tiles from
    per-XCD queues kept in a small workspace) instead of a workgroup per Q tile; same results."""
    L = lib()
    _require_gpu(q, k, v)
    if q.dtype not in (torch.float16, torch.bfloat16, torch.float32) + FP8_DTYPES:
        raise NotImplementedError(f"natten_amd fna_forward does not support {q.dtype}.")
    na_dim = len(kernel_size)
    scales = _scale_ptrs(q, k, q_scale, k_scale, v_scale)
    # 8-bit float operands are multiplied by the 8-bit matrix instruction; the result is bf16
    out = torch.empty(q.shape, dtype=torch.bfloat16 if q.dtype in FP8_DTYPES else q.dtype, device=q.device)
    lse = torch.empty(q.shape[:-1], dtype=torch.float32, device=q.device)
    with _on_device(q):
        rc = L.natten_amd_fna_forward(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
            DTYPE_CODES[q.dtype], na_dim, q.shape[0], q.shape[1], k.shape[1], q.shape[2], k.shape[2], q.shape[3],
            _i32(q_shape), _i32(kv_shape), _i32(qkv_shape), _i32(kernel_size), _i32(stride), _i32(dilation),
            _i32([1 if c else 0 for c in is_causal]), _i32(q_tile_shape), _i32(kv_tile_shape),
            float(scale), *scales, *_queue_workspace(q, run_persistent), _stream(q),
        )
    _check(rc)
    return out, lse


_QUEUE_WORKSPACES = {}


def _queue_workspace(like: Tensor, run_persistent: bool):
    """(flag, pointer, bytes) of the work-queue launch's workspace, allocated by the caller side as
    the reference's wrappers allocate theirs (src/natten/_libnatten/torch_wrappers.py:688-693).
    Always `run_persistent = 1`: the launch clears the counters itself (one small kernel ahead of
    the work-queue kernel), so nothing rests on what an earlier launch left in the block.  The C
    interface's `run_persistent = 2`, which skips that kernel for a caller who vouches for zeros,
    is not used from Python."""
    if not run_persistent:
        return 0, None, 0
    nbytes = int(lib().natten_amd_fna_forward_workspace_bytes())
    if torch.cuda.is_current_stream_capturing():
        # memory allocated under capture belongs to the graph: a block of its own
        ws = torch.empty(nbytes, dtype=torch.uint8, device=like.device)
        return 1, ws.data_ptr(), nbytes
    # one block per (device, stream): launches of one stream run one after the other
    key = (like.device.index, torch.cuda.current_stream(like.device).cuda_stream)
    ws = _QUEUE_WORKSPACES.get(key)
    if ws is None:
        ws = _QUEUE_WORKSPACES[key] = torch.empty(nbytes, dtype=torch.uint8, device=like.device)
    return 1, ws.data_ptr(), nbytes


def _tile_span_fits(token_layout, dilation, tile_shape, row_bytes: int) -> bool:
    """The kernels address the rows of a tile of the original tensors with 32-bit byte offsets
    from the tile's first row: the tile must span less than 2^31 bytes."""
    span, step = 0, 1
    for X, d, t in zip(reversed(token_layout), reversed(dilation), reversed(tile_shape)):
        span += (t - 1) * d * step
        step *= X
    return (span + 1) * row_bytes + 8192 < 2**31 - 1


def fused_layout_supported(qkv_shape, dilation, kv_tile_shape, row_bytes: int = 0, q_tile_shape=None,
                           dtype: Optional[torch.dtype] = None) -> bool:
    """Whether fna_forward_fused accepts this problem.  Always: (given `row_bytes` = heads_kv *
    head_dim * 2) a KV tile spans less than 2^31 bytes of the input.  When every extent is a multiple
    of dilation x KV tile no KV tile reaches past its dilation group.  Otherwise (`q_tile_shape`
    and `dtype` given) every dilation group must be at least a KV tile wide in every dimension, or
    the operands fp16 / bf16 with tiles of 128 x 64 tokens (the one instance that clamps)."""
    if not _tile_span_fits(qkv_shape, dilation, kv_tile_shape, row_bytes):
        return False
    if all(X % (d * t) == 0 for X, d, t in zip(qkv_shape, dilation, kv_tile_shape)):
        return True
    if q_tile_shape is None or dtype is None:
        return False
    if all(X // d >= t for X, d, t in zip(qkv_shape, dilation, kv_tile_shape)):
        return True  # (every kernel moves a tile that would reach past its group back to the group's end)
    if dtype not in (torch.float16, torch.bfloat16):
        return False
    q_tokens = kv_tokens = 1
    for tq, tk in zip(q_tile_shape, kv_tile_shape):
        q_tokens *= tq
        kv_tokens *= tk
    return q_tokens == 128 and kv_tokens == 64


def fna_forward_fused(
    q: Tensor, k: Tensor, v: Tensor,
    kernel_size, stride, dilation, is_causal, scale: float, q_tile_shape, kv_tile_shape,
    q_scale: Optional[Tensor] = None, k_scale: Optional[Tensor] = None, v_scale: Optional[Tensor] = None,
    run_persistent: bool = False, anchored_tiles: bool = True,
) -> Tuple[Tensor, Tensor]:
    """Original-layout q [B, *X, H, D], k/v [B, *X, Hkv, D] -> (out like q, lse float32 [B, *X, H]).
    anchored_tiles: lay the KV tiles of a Q tile out from the first key of its window instead of
    from multiples of the tile extent (fewer tiles; sums run in another order than on the permuted path)."""
    L = lib()
    _require_gpu(q, k, v)
    if q.dtype not in (torch.float16, torch.bfloat16) + FP8_DTYPES:
        raise NotImplementedError(f"natten_amd fna_forward_fused does not support {q.dtype}.")
    na_dim = len(kernel_size)
    qkv_shape = [int(x) for x in q.shape[1 : 1 + na_dim]]
    scales = _scale_ptrs(q, k, q_scale, k_scale, v_scale)
    out = torch.empty(q.shape, dtype=torch.bfloat16 if q.dtype in FP8_DTYPES else q.dtype, device=q.device)
    lse = torch.empty(q.shape[:-1], dtype=torch.float32, device=q.device)
    with _on_device(q):
        rc = L.natten_amd_fna_forward_fused(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
            DTYPE_CODES[q.dtype], na_dim, q.shape[0], q.shape[-2], k.shape[-2], q.shape[-1],
            _i32(qkv_shape), _i32(kernel_size), _i32(stride), _i32(dilation),
            _i32([1 if c else 0 for c in is_causal]), _i32(q_tile_shape), _i32(kv_tile_shape),
            float(scale), *scales, 1 if anchored_tiles else 0, *_queue_workspace(q, run_persistent), _stream(q),
        )
    _check(rc)
    return out, lse


def fna_forward_fused_split(
    q: Tensor, k: Tensor, v: Tensor,
    kernel_size, stride, dilation, is_causal, scale: float, q_tile_shape, kv_tile_shape,
    kv_splits: int, anchored_tiles: bool = True,
) -> Tuple[Tensor, Tensor]:
    """fna_forward_fused with the KV tiles of every Q tile dealt to `kv_splits` workgroups: returns
    the partial results (out_parts [kv_splits, B, *X, H, D], lse_parts float32 [kv_splits, B, *X, H]),
    each normalised over the keys of its own run of tiles (zeros and -inf where a run holds none of a
    query's keys); merge_parts combines them."""
    L = lib()
    _require_gpu(q, k, v)
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError(f"natten_amd fna_forward_fused_split does not support {q.dtype}.")
    na_dim = len(kernel_size)
    qkv_shape = [int(x) for x in q.shape[1 : 1 + na_dim]]
    out = torch.empty((kv_splits, *q.shape), dtype=q.dtype, device=q.device)
    lse = torch.empty((kv_splits, *q.shape[:-1]), dtype=torch.float32, device=q.device)
    with _on_device(q):
        rc = L.natten_amd_fna_forward_fused_split(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
            DTYPE_CODES[q.dtype], na_dim, q.shape[0], q.shape[-2], k.shape[-2], q.shape[-1],
            _i32(qkv_shape), _i32(kernel_size), _i32(stride), _i32(dilation),
            _i32([1 if c else 0 for c in is_causal]), _i32(q_tile_shape), _i32(kv_tile_shape),
            float(scale), 1 if anchored_tiles else 0, int(kv_splits), _stream(q),
        )
    _check(rc)
    return out, lse


def fna_forward_fused_static(
    q: Tensor, k: Tensor, v: Tensor, out: Tensor, lse: Tensor,
    kernel_size, stride, dilation, is_causal, scale: float, q_tile_shape, kv_tile_shape,
) -> None:
    """fna_forward_fused as a work-queue launch whose queues live in the library's own device
    image: the call allocates nothing, so the caller passes the results' buffers too
    (out like q, lse float32 [B, *X, H]).  For callers that cannot allocate; calls that overlap
    in time on one GPU must not be made."""
    L = lib()
    _require_gpu(q, k, v, out, lse)
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError(f"natten_amd fna_forward_fused_static does not support {q.dtype}.")
    if out.shape != q.shape or out.dtype != q.dtype or not out.is_contiguous():
        raise ValueError("out must be a contiguous tensor of q's shape and dtype.")
    if lse.shape != q.shape[:-1] or lse.dtype != torch.float32 or not lse.is_contiguous():
        raise ValueError("lse must be a contiguous float32 tensor of q's shape without the last dimension.")
    na_dim = len(kernel_size)
    qkv_shape = [int(x) for x in q.shape[1 : 1 + na_dim]]
    with _on_device(q):
        rc = L.natten_amd_fna_forward_fused_static(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
            DTYPE_CODES[q.dtype], na_dim, q.shape[0], q.shape[-2], k.shape[-2], q.shape[-1],
            _i32(qkv_shape), _i32(kernel_size), _i32(stride), _i32(dilation),
            _i32([1 if c else 0 for c in is_causal]), _i32(q_tile_shape), _i32(kv_tile_shape),
            float(scale), None, None, None, _stream(q),
        )
    _check(rc)


def attention_forward(
    q: Tensor, k: Tensor, v: Tensor, is_causal: bool, scale: float,
    q_scale: Optional[Tensor] = None, k_scale: Optional[Tensor] = None, v_scale: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor]:
    """Dense attention q [B, S, H, D], k/v [B, Skv, Hkv, D] -> (out, lse float32 [B, S, H])."""
    L = lib()
    _require_gpu(q, k, v)
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError(f"natten_amd attention_forward does not support {q.dtype}.")
    scales = _scale_ptrs(q, k, q_scale, k_scale, v_scale)
    out = torch.empty_like(q)
    lse = torch.empty(q.shape[:-1], dtype=torch.float32, device=q.device)
    with _on_device(q):
        rc = L.natten_amd_attention_forward(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), DTYPE_CODES[q.dtype],
            q.shape[0], q.shape[1], k.shape[1], q.shape[2], k.shape[2], q.shape[3], 1 if is_causal else 0,
            float(scale), *scales, _stream(q),
        )
    _check(rc)
    return out, lse


def attention_forward_varlen(
    q: Tensor, k: Tensor, v: Tensor, cumulative_seqlen_q: Tensor, cumulative_seqlen_kv: Tensor,
    max_seqlen_q: int, max_seqlen_kv: int, is_causal: bool, scale: float,
    q_scale: Optional[Tensor] = None, k_scale: Optional[Tensor] = None, v_scale: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor]:
    """Sequence-packed dense attention: q [1, total_q, H, D], k/v [1, total_kv, Hkv, D], int32
    device arrays of cumulative lengths (leading 0) -> (out, lse float32 [1, total_q, H]).  Rows
    that belong to no sequence come back as zeros."""
    L = lib()
    _require_gpu(q, k, v, cumulative_seqlen_q, cumulative_seqlen_kv)
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError(f"natten_amd attention_forward_varlen does not support {q.dtype}.")
    if q.shape[0] != 1 or k.shape[0] != 1:
        raise ValueError("variable-length attention takes the sequence-packed layout (batch = 1).")
    for c in (cumulative_seqlen_q, cumulative_seqlen_kv):
        if c.dtype != torch.int32 or c.dim() != 1 or not c.is_contiguous():
            raise ValueError("cumulative sequence lengths must be contiguous 1-D int32 tensors.")
    if cumulative_seqlen_q.shape[0] != cumulative_seqlen_kv.shape[0] or cumulative_seqlen_q.shape[0] < 2:
        raise ValueError("cumulative sequence lengths must match in size and hold at least 2 entries.")
    scales = _scale_ptrs(q, k, q_scale, k_scale, v_scale)
    out = torch.zeros_like(q)
    lse = torch.zeros(q.shape[:-1], dtype=torch.float32, device=q.device)
    with _on_device(q):
        rc = L.natten_amd_attention_forward_varlen(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), DTYPE_CODES[q.dtype],
            cumulative_seqlen_q.shape[0] - 1, q.shape[1], k.shape[1], int(max_seqlen_q), int(max_seqlen_kv),
            q.shape[2], k.shape[2], q.shape[3], cumulative_seqlen_q.data_ptr(), cumulative_seqlen_kv.data_ptr(),
            1 if is_causal else 0, float(scale), *scales, _stream(q),
        )
    _check(rc)
    return out, lse


def window(query: int, kernel_size: int, stride: int, extent: int, is_causal: bool) -> Tuple[int, int]:
    """[start, end) of the key coordinates a query coordinate attends along one dimension (host
    arithmetic only, the routine of the forward kernels' set-up)."""
    st, en = ctypes.c_int32(), ctypes.c_int32()
    _check(lib().natten_amd_window(int(query), int(kernel_size), int(stride), int(extent), int(bool(is_causal)),
                                   ctypes.addressof(st), ctypes.addressof(en)))
    return st.value, en.value


def tile_key_mask(kv_tile_shape, lo, hi) -> int:
    """Bit i set = key i of a 64-key KV tile (dimension 0 fastest) has in-tile coordinates inside
    [lo, hi) along every dimension (host arithmetic only, the rows of the kernels' element mask)."""
    pad = lambda x, fill: list(x) + [fill] * (3 - len(x))
    m = ctypes.c_uint64()
    _check(lib().natten_amd_tile_key_mask(_i32(pad(kv_tile_shape, 1)), _i32(pad(lo, 0)), _i32(pad(hi, 1)),
                                          ctypes.addressof(m)))
    return m.value


def fully_block_sparse(qkv_shape, kernel_size, stride, dilation, is_causal, q_tile_shape, kv_tile_shape,
                       anchored_tiles: bool = True) -> bool:
    """Whether the one-launch forward runs this problem with the instance that holds no mask code
    (host arithmetic only)."""
    r = ctypes.c_int32()
    _check(lib().natten_amd_fna_fully_block_sparse(
        len(qkv_shape), _i32(qkv_shape), _i32(kernel_size), _i32(stride), _i32(dilation),
        _i32([1 if c else 0 for c in is_causal]), _i32(q_tile_shape), _i32(kv_tile_shape), 1 if anchored_tiles else 0,
        ctypes.addressof(r)))
    return bool(r.value)


def wave_box(qkv_shape, kernel_size, stride, dilation, is_causal, q_tile_shape, kv_tile_shape,
             anchored_tiles: bool = True) -> Tuple[int, ...]:
    """The box of 32 queries that one wave of the 16-bit forward kernels holds for this problem
    (host arithmetic only)."""
    box = (ctypes.c_int32 * len(qkv_shape))()
    _check(lib().natten_amd_fna_wave_box(
        len(qkv_shape), _i32(qkv_shape), _i32(kernel_size), _i32(stride), _i32(dilation),
        _i32([1 if c else 0 for c in is_causal]), _i32(q_tile_shape), _i32(kv_tile_shape), 1 if anchored_tiles else 0,
        ctypes.addressof(box)))
    return tuple(int(x) for x in box)


def query_range(key_first: int, key_last: int, kernel_size: int, stride: int, extent: int, num_queries: int,
                is_causal: bool) -> Tuple[int, int]:
    """(first, last) query coordinate whose window meets keys key_first .. key_last (host arithmetic only)."""
    first, last = ctypes.c_int32(), ctypes.c_int32()
    _check(lib().natten_amd_query_range(int(key_first), int(key_last), int(kernel_size), int(stride), int(extent),
                                        int(num_queries), 1 if is_causal else 0, ctypes.byref(first),
                                        ctypes.byref(last)))
    return first.value, last.value


def compute_delta(out: Tensor, d_out: Tensor) -> Tensor:
    """rowsum(out * d_out) over the last dimension, float32, shape out.shape[:-1]."""
    L = lib()
    _require_gpu(out, d_out)
    if out.dtype not in (torch.float16, torch.bfloat16) or d_out.dtype != out.dtype or d_out.shape != out.shape:
        raise ValueError("compute_delta needs two fp16 / bf16 tensors of the same shape and dtype.")
    delta = torch.empty(out.shape[:-1], dtype=torch.float32, device=out.device)
    with _on_device(out):
        rc = L.natten_amd_compute_delta(out.data_ptr(), d_out.data_ptr(), delta.data_ptr(), DTYPE_CODES[out.dtype],
                                        delta.numel(), out.shape[-1], _stream(out))
    _check(rc)
    return delta


def fna_backward(
    q: Tensor, k: Tensor, v: Tensor, d_out: Tensor, lse: Tensor, delta: Tensor, kernel_size, stride, dilation,
    is_causal, scale: float, q_shape, kv_shape, qkv_shape, q_tile_shape, kv_tile_shape,
) -> Tuple[Tensor, Tensor, Tensor]:
    """Backward on token-permuted operands (128-token tiles on both sides) -> (dq, dk, dv).
    lse, delta: [batch, seqlen_q, heads_q] as the permute gives them; the kernels take them head-major."""
    L = lib()
    lse, delta = lse.transpose(1, 2).contiguous(), delta.transpose(1, 2).contiguous()
    _require_gpu(q, k, v, d_out, lse, delta)
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError(f"natten_amd fna_backward does not support {q.dtype}.")
    if lse.dtype != torch.float32 or delta.dtype != torch.float32:
        raise ValueError("lse and delta must be float32.")
    na_dim = len(kernel_size)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    with _on_device(q):
        rc = L.natten_amd_fna_backward(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), d_out.data_ptr(), lse.data_ptr(), delta.data_ptr(),
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dq.data_ptr(), DTYPE_CODES[q.dtype], na_dim, q.shape[0], q.shape[1],
            k.shape[1], q.shape[2], k.shape[2], q.shape[3], _i32(q_shape), _i32(kv_shape), _i32(qkv_shape),
            _i32(kernel_size), _i32(stride), _i32(dilation), _i32([1 if c else 0 for c in is_causal]),
            _i32(q_tile_shape), _i32(kv_tile_shape), float(scale), _stream(q),
        )
    _check(rc)
    return dq, dk, dv


def backward_fused_layout_supported(token_layout, dilation, q_tile_shape, kv_tile_shape, row_bytes: int = 0) -> bool:
    """Whether the backward kernels can work on the original tensors: every dilation group at least
    one tile wide (either side's) in every dimension, and (given `row_bytes` = heads_q * head_dim * 2)
    tiles that span less than 2^31 bytes."""
    return (
        all(X // d >= tq and X // d >= tk
            for X, d, tq, tk in zip(token_layout, dilation, q_tile_shape, kv_tile_shape))
        and _tile_span_fits(token_layout, dilation, q_tile_shape, row_bytes)
        and _tile_span_fits(token_layout, dilation, kv_tile_shape, row_bytes)
    )


def fna_backward_fused(
    q: Tensor, k: Tensor, v: Tensor, d_out: Tensor, lse: Tensor, delta: Tensor, kernel_size, stride, dilation,
    is_causal, scale: float, q_tile_shape, kv_tile_shape, kv_role_q_tile_shape=None, kv_role_kv_tile_shape=None,
) -> Tuple[Tensor, Tensor, Tensor]:
    """Backward on the original tensors [B, *X, H, D] (lse, delta [B, *X, H]) -> (dq, dk, dv).
    kv_role_*_tile_shape: tile shapes of the launch that forms dk and dv, when they differ from those
    of the dq launch (q_tile_shape, kv_tile_shape)."""
    L = lib()
    na_dim = len(kernel_size)
    B, H = q.shape[0], q.shape[-2]
    lse = lse.reshape(B, -1, H).transpose(1, 2).contiguous()
    delta = delta.reshape(B, -1, H).transpose(1, 2).contiguous()
    _require_gpu(q, k, v, d_out, lse, delta)
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError(f"natten_amd fna_backward_fused does not support {q.dtype}.")
    if lse.dtype != torch.float32 or delta.dtype != torch.float32:
        raise ValueError("lse and delta must be float32.")
    if (kv_role_q_tile_shape is None) != (kv_role_kv_tile_shape is None):
        raise ValueError("kv_role_q_tile_shape and kv_role_kv_tile_shape must be given together.")
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    same = kv_role_q_tile_shape is None or (
        tuple(kv_role_q_tile_shape) == tuple(q_tile_shape) and tuple(kv_role_kv_tile_shape) == tuple(kv_tile_shape))
    # The dk / dv launch streams the queries as the forward kernel multiplied them (scaled, rounded
    # once) from a workspace of q's size that the call fills first; dq serves as that workspace, so
    # the launch that writes dq comes last.
    launches = [(3, q_tile_shape, kv_tile_shape)] if same else [
        (2, kv_role_q_tile_shape, kv_role_kv_tile_shape), (1, q_tile_shape, kv_tile_shape)]
    with _on_device(q):
        for roles, qt, kt in launches:
            rc = L.natten_amd_fna_backward_fused(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), d_out.data_ptr(), lse.data_ptr(), delta.data_ptr(),
                dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dq.data_ptr(), DTYPE_CODES[q.dtype], na_dim, B, H, k.shape[-2],
                q.shape[-1], _i32(q.shape[1 : 1 + na_dim]), _i32(kernel_size), _i32(stride), _i32(dilation),
                _i32([1 if c else 0 for c in is_causal]), _i32(qt), _i32(kt), float(scale), roles, _stream(q),
            )
            _check(rc)
    return dq, dk, dv


def attention_backward(
    q: Tensor, k: Tensor, v: Tensor, d_out: Tensor, lse: Tensor, delta: Tensor, seqlen_q: int, seqlen_kv: int,
    is_causal: bool, scale: float,
) -> Tuple[Tensor, Tensor, Tensor]:
    """Dense attention backward on operands zero-padded to multiples of 128 rows -> (dq, dk, dv), padded alike.
    lse, delta: [batch, padded seqlen_q, heads_q]; the kernels take them head-major."""
    L = lib()
    lse, delta = lse.transpose(1, 2).contiguous(), delta.transpose(1, 2).contiguous()
    _require_gpu(q, k, v, d_out, lse, delta)
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError(f"natten_amd attention_backward does not support {q.dtype}.")
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    with _on_device(q):
        rc = L.natten_amd_attention_backward(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), d_out.data_ptr(), lse.data_ptr(), delta.data_ptr(),
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dq.data_ptr(), DTYPE_CODES[q.dtype], q.shape[0], int(seqlen_q),
            int(seqlen_kv), q.shape[1], k.shape[1], q.shape[2], k.shape[2], q.shape[3], 1 if is_causal else 0,
            float(scale), _stream(q),
        )
    _check(rc)
    return dq, dk, dv


def attention_backward_varlen(
    q: Tensor, k: Tensor, v: Tensor, d_out: Tensor, lse: Tensor, delta: Tensor, cu_q: Tensor, cu_kv: Tensor,
    padded_cu_q: Tensor, padded_cu_kv: Tensor, max_seqlen_q: int, max_seqlen_kv: int, is_causal: bool, scale: float,
) -> Tuple[Tensor, Tensor, Tensor]:
    """Dense attention backward of a sequence-packed batch whose sequences are each zero-padded to
    a multiple of 128 rows -> (dq, dk, dv) in the same padded packing.  q, d_out [1, rows_q, H, D];
    k, v [1, rows_kv, Hkv, D]; lse, delta [1, rows_q, H] (the kernels take them head-major); the
    four cumulative arrays are device int32 [sequences + 1].  Rows outside every sequence's padded
    range are left unwritten."""
    L = lib()
    lse, delta = lse.transpose(1, 2).contiguous(), delta.transpose(1, 2).contiguous()
    _require_gpu(q, k, v, d_out, lse, delta, cu_q, cu_kv, padded_cu_q, padded_cu_kv)
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError(f"natten_amd attention_backward_varlen does not support {q.dtype}.")
    cums = (cu_q, cu_kv, padded_cu_q, padded_cu_kv)
    if any(c.dtype != torch.int32 or c.dim() != 1 or c.numel() != cu_q.numel() or not c.is_contiguous() for c in cums):
        raise ValueError("cumulative sequence lengths must be contiguous int32 vectors of one length.")
    if cu_q.numel() < 2 or q.shape[0] != 1 or k.shape[0] != 1:
        raise ValueError("sequence-packed operands have batch 1 and at least one sequence.")
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    with _on_device(q):
        rc = L.natten_amd_attention_backward_varlen(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), d_out.data_ptr(), lse.data_ptr(), delta.data_ptr(),
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dq.data_ptr(), DTYPE_CODES[q.dtype], cu_q.numel() - 1, q.shape[1], k.shape[1],
            cu_q.data_ptr(), cu_kv.data_ptr(), padded_cu_q.data_ptr(), padded_cu_kv.data_ptr(), int(max_seqlen_q),
            int(max_seqlen_kv), q.shape[2], k.shape[2], q.shape[3], 1 if is_causal else 0, float(scale), _stream(q),
        )
    _check(rc)
    return dq, dk, dv


def _ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


def token_permute(x: Tensor, tile_shape, dilation, flip_tiled_dims: bool, widen: bool = False) -> Tensor:
    """[B, *X, H, Dh] -> [B * prod(dilation), prod(ceil(ceil(X/t)/d) * t), H, Dh], zero padded.

    widen=True (8-bit float input only) writes the exact bf16 values instead of the raw bytes."""
    L = lib()
    _require_gpu(x)
    if widen and x.dtype not in FP8_DTYPES:
        raise ValueError(f"token_permute(widen=True) needs an 8-bit float tensor, got {x.dtype}.")
    na_dim = x.dim() - 3
    layout = [int(s) for s in x.shape[1 : 1 + na_dim]]
    post = [_ceil_div(_ceil_div(X, t), d) * t for X, t, d in zip(layout, tile_shape, dilation)]
    groups = 1
    seqlen = 1
    for d, p in zip(dilation, post):
        groups *= d
        seqlen *= p
    out_dtype = torch.bfloat16 if widen else x.dtype
    out = torch.empty((x.shape[0] * groups, seqlen, x.shape[-2], x.shape[-1]), dtype=out_dtype, device=x.device)
    if widen:
        with _on_device(x):
            rc = L.natten_amd_token_permute_widen(
                x.data_ptr(), out.data_ptr(), DTYPE_CODES[x.dtype], na_dim, x.shape[0], x.shape[-2], x.shape[-1],
                _i32(layout), _i32(tile_shape), _i32(dilation), 1 if flip_tiled_dims else 0, _stream(x),
            )
        _check(rc)
        return out
    with _on_device(x):
        rc = L.natten_amd_token_permute(
            x.data_ptr(), out.data_ptr(), x.element_size(), na_dim, x.shape[0], x.shape[-2], x.shape[-1],
            _i32(layout), _i32(tile_shape), _i32(dilation), 1 if flip_tiled_dims else 0, _stream(x),
        )
    _check(rc)
    return out


def token_unpermute(y: Tensor, token_layout, tile_shape, dilation, flip_tiled_dims: bool) -> Tensor:
    """Inverse of token_permute: [B*G, S', H, Dh] -> [B, *token_layout, H, Dh]."""
    L = lib()
    _require_gpu(y)
    na_dim = len(token_layout)
    groups = 1
    seqlen = 1
    for X, t, d in zip(token_layout, tile_shape, dilation):
        groups *= d
        seqlen *= _ceil_div(_ceil_div(X, t), d) * t
    if y.dim() != 4 or y.shape[0] % groups != 0 or y.shape[1] != seqlen:
        raise RuntimeError(
            f"token_unpermute: tensor of shape {tuple(y.shape)} does not match token layout {tuple(token_layout)}, "
            f"tile shape {tuple(tile_shape)}, dilation {tuple(dilation)} (expected [B*{groups}, {seqlen}, H, D])."
        )
    batch = y.shape[0] // groups
    out = torch.empty((batch, *token_layout, y.shape[-2], y.shape[-1]), dtype=y.dtype, device=y.device)
    with _on_device(y):
        rc = L.natten_amd_token_unpermute(
            y.data_ptr(), out.data_ptr(), y.element_size(), na_dim, batch, y.shape[-2], y.shape[-1],
            _i32(token_layout), _i32(tile_shape), _i32(dilation), 1 if flip_tiled_dims else 0, _stream(y),
        )
    _check(rc)
    return out


def merge_two(o0: Tensor, lse0: Tensor, o1: Tensor, lse1: Tensor) -> Tuple[Tensor, Tensor]:
    """Merge two partial attentions [B, S, H, D] with float32 LSE [B, S, H]."""
    L = lib()
    _require_gpu(o0, lse0, o1, lse1)
    if o0.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise NotImplementedError(f"natten_amd merge does not support {o0.dtype}.")
    out = torch.empty_like(o0)
    lse = torch.empty_like(lse0)
    rows = lse0.numel()
    with _on_device(o0):
        rc = L.natten_amd_merge_attentions(
            o0.data_ptr(), lse0.data_ptr(), o1.data_ptr(), lse1.data_ptr(), out.data_ptr(), lse.data_ptr(),
            DTYPE_CODES[o0.dtype], rows, o0.shape[-1], _stream(o0),
        )
    _check(rc)
    return out, lse


def merge_parts(out_parts: Tensor, lse_parts: Tensor) -> Tuple[Tensor, Tensor]:
    """Merge the partial attentions out_parts [n, ..., D] with float32 LSE lse_parts [n, ...] (the
    layout fna_forward_fused_split returns) in one launch, float32 arithmetic, one rounding."""
    L = lib()
    _require_gpu(out_parts, lse_parts)
    if out_parts.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise NotImplementedError(f"natten_amd merge does not support {out_parts.dtype}.")
    if lse_parts.dtype != torch.float32 or lse_parts.shape != out_parts.shape[:-1]:
        raise ValueError("lse_parts must be float32 of out_parts' shape without the last dimension.")
    if not (out_parts.is_contiguous() and lse_parts.is_contiguous()):
        raise ValueError("out_parts and lse_parts must be contiguous.")
    out = torch.empty(out_parts.shape[1:], dtype=out_parts.dtype, device=out_parts.device)
    lse = torch.empty(lse_parts.shape[1:], dtype=torch.float32, device=out_parts.device)
    with _on_device(out_parts):
        rc = L.natten_amd_merge_attention_parts(
            out_parts.data_ptr(), lse_parts.data_ptr(), out_parts.shape[0], out.data_ptr(), lse.data_ptr(),
            DTYPE_CODES[out_parts.dtype], lse.numel(), out_parts.shape[-1], _stream(out_parts),
        )
    _check(rc)
    return out, lse


def mfma_probe(random_operands: bool = True, iters: int = 20000, fma_per_mfma: int = 0, device="cuda:0"):
    """Sustained bf16 MFMA rate of the device: returns (TFLOP/s, shader clock in GHz)."""
    L = lib()
    dev = torch.device(device)
    n = 256 * 256 * 64  # bf16 values
    if random_operands:
        gen = torch.Generator().manual_seed(0)
        ops = torch.randn(n, generator=gen).to(torch.bfloat16).to(dev)
    else:
        ops = torch.full((n,), 0.25, dtype=torch.bfloat16, device=dev)
    sink = torch.empty(256 * 256, dtype=torch.float32, device=dev)
    clocks = torch.zeros(2 * 256, dtype=torch.int64, device=dev)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def launch(k):
        with torch.cuda.device(dev):
            _check(L.natten_amd_mfma_probe(ops.data_ptr(), sink.data_ptr(), clocks.data_ptr(), k, fma_per_mfma,
                                           torch.cuda.current_stream(dev).cuda_stream))

    launch(max(iters // 20, 1))
    torch.cuda.synchronize(dev)
    e0.record()
    launch(iters)
    e1.record()
    torch.cuda.synchronize(dev)
    ms = e0.elapsed_time(e1)
    c = clocks.cpu().view(256, 2).double()
    ghz = float(c[:, 0].sum() / (c[:, 1].sum() * 10.0))
    flops = 256.0 * 4 * iters * 16 * 32768
    return flops / ms / 1e9, ghz
