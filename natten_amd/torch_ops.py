"""The native entry points as torch custom operators, for tracing compilers.

Counterpart of the reference's src/natten/_libnatten/torch_wrappers.py:98-103, :657-751,
:1373-1503 (custom_op + register_fake per native function).  In eager mode the drivers call
the ctypes binding directly (a custom operator costs some microseconds of dispatch per call);
under `torch.compile` they go through these operators, whose fake implementations give the
tracer shapes and dtypes without touching the device.
"""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch
from torch import Tensor

from . import _lib

_FP8 = _lib.FP8_DTYPES


def _out_dtype(q: Tensor) -> torch.dtype:
    return torch.bfloat16 if q.dtype in _FP8 else q.dtype


@torch.library.custom_op("natten_amd::fna_forward", mutates_args=(), device_types="cuda")
def _fna_forward_op(
    q: Tensor, k: Tensor, v: Tensor, kernel_size: List[int], stride: List[int], dilation: List[int],
    is_causal: List[bool], scale: float, q_shape: List[int], kv_shape: List[int], qkv_shape: List[int],
    q_tile_shape: List[int], kv_tile_shape: List[int], q_scale: Optional[Tensor], k_scale: Optional[Tensor],
    v_scale: Optional[Tensor], run_persistent: bool,
) -> Tuple[Tensor, Tensor]:
    return _lib.fna_forward(q, k, v, kernel_size, stride, dilation, is_causal, scale, q_shape, kv_shape, qkv_shape,
                            q_tile_shape, kv_tile_shape, q_scale=q_scale, k_scale=k_scale, v_scale=v_scale,
                            run_persistent=run_persistent)


@_fna_forward_op.register_fake
def _(q, k, v, kernel_size, stride, dilation, is_causal, scale, q_shape, kv_shape, qkv_shape, q_tile_shape,
      kv_tile_shape, q_scale, k_scale, v_scale, run_persistent):
    return q.new_empty(q.shape, dtype=_out_dtype(q)), q.new_empty(q.shape[:-1], dtype=torch.float32)


@torch.library.custom_op("natten_amd::fna_forward_fused", mutates_args=(), device_types="cuda")
def _fna_forward_fused_op(
    q: Tensor, k: Tensor, v: Tensor, kernel_size: List[int], stride: List[int], dilation: List[int],
    is_causal: List[bool], scale: float, q_tile_shape: List[int], kv_tile_shape: List[int],
    q_scale: Optional[Tensor], k_scale: Optional[Tensor], v_scale: Optional[Tensor], run_persistent: bool,
    anchored_tiles: bool,
) -> Tuple[Tensor, Tensor]:
    return _lib.fna_forward_fused(q, k, v, kernel_size, stride, dilation, is_causal, scale, q_tile_shape,
                                  kv_tile_shape, q_scale=q_scale, k_scale=k_scale, v_scale=v_scale,
                                  run_persistent=run_persistent, anchored_tiles=anchored_tiles)


@_fna_forward_fused_op.register_fake
def _(q, k, v, kernel_size, stride, dilation, is_causal, scale, q_tile_shape, kv_tile_shape, q_scale, k_scale, v_scale,
      run_persistent, anchored_tiles):
    return q.new_empty(q.shape, dtype=_out_dtype(q)), q.new_empty(q.shape[:-1], dtype=torch.float32)


@torch.library.custom_op("natten_amd::attention_forward", mutates_args=(), device_types="cuda")
def _attention_forward_op(
    q: Tensor, k: Tensor, v: Tensor, is_causal: bool, scale: float, q_scale: Optional[Tensor],
    k_scale: Optional[Tensor], v_scale: Optional[Tensor],
) -> Tuple[Tensor, Tensor]:
    return _lib.attention_forward(q, k, v, is_causal, scale, q_scale=q_scale, k_scale=k_scale, v_scale=v_scale)


@_attention_forward_op.register_fake
def _(q, k, v, is_causal, scale, q_scale, k_scale, v_scale):
    return torch.empty_like(q), q.new_empty(q.shape[:-1], dtype=torch.float32)


@torch.library.custom_op("natten_amd::attention_forward_varlen", mutates_args=(), device_types="cuda")
def _attention_forward_varlen_op(
    q: Tensor, k: Tensor, v: Tensor, cumulative_seqlen_q: Tensor, cumulative_seqlen_kv: Tensor,
    max_seqlen_q: int, max_seqlen_kv: int, is_causal: bool, scale: float, q_scale: Optional[Tensor],
    k_scale: Optional[Tensor], v_scale: Optional[Tensor],
) -> Tuple[Tensor, Tensor]:
    return _lib.attention_forward_varlen(q, k, v, cumulative_seqlen_q, cumulative_seqlen_kv, max_seqlen_q,
                                         max_seqlen_kv, is_causal, scale, q_scale=q_scale, k_scale=k_scale,
                                         v_scale=v_scale)


@_attention_forward_varlen_op.register_fake
def _(q, k, v, cumulative_seqlen_q, cumulative_seqlen_kv, max_seqlen_q, max_seqlen_kv, is_causal, scale, q_scale,
      k_scale, v_scale):
    return torch.empty_like(q), q.new_empty(q.shape[:-1], dtype=torch.float32)


@torch.library.custom_op("natten_amd::compute_delta", mutates_args=(), device_types="cuda")
def _compute_delta_op(out: Tensor, d_out: Tensor) -> Tensor:
    return _lib.compute_delta(out, d_out)


@_compute_delta_op.register_fake
def _(out, d_out):
    return out.new_empty(out.shape[:-1], dtype=torch.float32)


@torch.library.custom_op("natten_amd::fna_backward", mutates_args=(), device_types="cuda")
def _fna_backward_op(
    q: Tensor, k: Tensor, v: Tensor, d_out: Tensor, lse: Tensor, delta: Tensor, kernel_size: List[int],
    stride: List[int], dilation: List[int], is_causal: List[bool], scale: float, q_shape: List[int],
    kv_shape: List[int], qkv_shape: List[int], q_tile_shape: List[int], kv_tile_shape: List[int],
) -> Tuple[Tensor, Tensor, Tensor]:
    return _lib.fna_backward(q, k, v, d_out, lse, delta, kernel_size, stride, dilation, is_causal, scale, q_shape,
                             kv_shape, qkv_shape, q_tile_shape, kv_tile_shape)


@_fna_backward_op.register_fake
def _(q, k, v, d_out, lse, delta, kernel_size, stride, dilation, is_causal, scale, q_shape, kv_shape, qkv_shape,
      q_tile_shape, kv_tile_shape):
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)


@torch.library.custom_op("natten_amd::fna_backward_fused", mutates_args=(), device_types="cuda")
def _fna_backward_fused_op(
    q: Tensor, k: Tensor, v: Tensor, d_out: Tensor, lse: Tensor, delta: Tensor, kernel_size: List[int],
    stride: List[int], dilation: List[int], is_causal: List[bool], scale: float, q_tile_shape: List[int],
    kv_tile_shape: List[int], kv_role_q_tile_shape: Optional[List[int]] = None,
    kv_role_kv_tile_shape: Optional[List[int]] = None,
) -> Tuple[Tensor, Tensor, Tensor]:
    return _lib.fna_backward_fused(q, k, v, d_out, lse, delta, kernel_size, stride, dilation, is_causal, scale,
                                   q_tile_shape, kv_tile_shape, kv_role_q_tile_shape, kv_role_kv_tile_shape)


@_fna_backward_fused_op.register_fake
def _(q, k, v, d_out, lse, delta, kernel_size, stride, dilation, is_causal, scale, q_tile_shape, kv_tile_shape,
      kv_role_q_tile_shape=None, kv_role_kv_tile_shape=None):
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)


@torch.library.custom_op("natten_amd::attention_backward", mutates_args=(), device_types="cuda")
def _attention_backward_op(
    q: Tensor, k: Tensor, v: Tensor, d_out: Tensor, lse: Tensor, delta: Tensor, seqlen_q: int, seqlen_kv: int,
    is_causal: bool, scale: float,
) -> Tuple[Tensor, Tensor, Tensor]:
    return _lib.attention_backward(q, k, v, d_out, lse, delta, seqlen_q, seqlen_kv, is_causal, scale)


@_attention_backward_op.register_fake
def _(q, k, v, d_out, lse, delta, seqlen_q, seqlen_kv, is_causal, scale):
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)


@torch.library.custom_op("natten_amd::attention_backward_varlen", mutates_args=(), device_types="cuda")
def _attention_backward_varlen_op(
    q: Tensor, k: Tensor, v: Tensor, d_out: Tensor, lse: Tensor, delta: Tensor, cu_q: Tensor, cu_kv: Tensor,
    padded_cu_q: Tensor, padded_cu_kv: Tensor, max_seqlen_q: int, max_seqlen_kv: int, is_causal: bool, scale: float,
) -> Tuple[Tensor, Tensor, Tensor]:
    return _lib.attention_backward_varlen(q, k, v, d_out, lse, delta, cu_q, cu_kv, padded_cu_q, padded_cu_kv,
                                          max_seqlen_q, max_seqlen_kv, is_causal, scale)


@_attention_backward_varlen_op.register_fake
def _(q, k, v, d_out, lse, delta, cu_q, cu_kv, padded_cu_q, padded_cu_kv, max_seqlen_q, max_seqlen_kv, is_causal, scale):
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)


def _permuted_shape(x: Tensor, tile_shape: List[int], dilation: List[int]) -> List[int]:
    na_dim = x.dim() - 3
    groups, seqlen = 1, 1
    for X, t, d in zip(x.shape[1 : 1 + na_dim], tile_shape, dilation):
        groups *= d
        seqlen *= -(-(-(-X // t)) // d) * t
    return [x.shape[0] * groups, seqlen, x.shape[-2], x.shape[-1]]


@torch.library.custom_op("natten_amd::token_permute", mutates_args=(), device_types="cuda")
def _token_permute_op(x: Tensor, tile_shape: List[int], dilation: List[int], flip_tiled_dims: bool, widen: bool) -> Tensor:
    return _lib.token_permute(x, tile_shape, dilation, flip_tiled_dims, widen=widen)


@_token_permute_op.register_fake
def _(x, tile_shape, dilation, flip_tiled_dims, widen):
    return x.new_empty(_permuted_shape(x, tile_shape, dilation), dtype=torch.bfloat16 if widen else x.dtype)


@torch.library.custom_op("natten_amd::token_unpermute", mutates_args=(), device_types="cuda")
def _token_unpermute_op(
    y: Tensor, token_layout: List[int], tile_shape: List[int], dilation: List[int], flip_tiled_dims: bool
) -> Tensor:
    return _lib.token_unpermute(y, token_layout, tile_shape, dilation, flip_tiled_dims)


@_token_unpermute_op.register_fake
def _(y, token_layout, tile_shape, dilation, flip_tiled_dims):
    groups = 1
    for d in dilation:
        groups *= d
    return y.new_empty([y.shape[0] // groups, *token_layout, y.shape[-2], y.shape[-1]])


@torch.library.custom_op("natten_amd::merge_two", mutates_args=(), device_types="cuda")
def _merge_two_op(o0: Tensor, lse0: Tensor, o1: Tensor, lse1: Tensor) -> Tuple[Tensor, Tensor]:
    return _lib.merge_two(o0, lse0, o1, lse1)


@_merge_two_op.register_fake
def _(o0, lse0, o1, lse1):
    return torch.empty_like(o0), torch.empty_like(lse0)


def _tracing() -> bool:
    return torch.compiler.is_compiling()


def _ints(t) -> List[int]:
    return [int(x) for x in t]


# ---- what the drivers call -------------------------------------------------------------------------

def fna_forward(q, k, v, kernel_size, stride, dilation, is_causal, scale, q_shape, kv_shape, qkv_shape, q_tile_shape,
                kv_tile_shape, q_scale=None, k_scale=None, v_scale=None, run_persistent=False):
    if _tracing():
        return _fna_forward_op(q, k, v, _ints(kernel_size), _ints(stride), _ints(dilation),
                               [bool(c) for c in is_causal], float(scale), _ints(q_shape), _ints(kv_shape),
                               _ints(qkv_shape), _ints(q_tile_shape), _ints(kv_tile_shape), q_scale, k_scale, v_scale,
                               bool(run_persistent))
    return _lib.fna_forward(q, k, v, kernel_size, stride, dilation, is_causal, scale, q_shape, kv_shape, qkv_shape,
                            q_tile_shape, kv_tile_shape, q_scale=q_scale, k_scale=k_scale, v_scale=v_scale,
                            run_persistent=run_persistent)


def fna_forward_fused(q, k, v, kernel_size, stride, dilation, is_causal, scale, q_tile_shape, kv_tile_shape,
                      q_scale=None, k_scale=None, v_scale=None, run_persistent=False, anchored_tiles=True):
    if _tracing():
        return _fna_forward_fused_op(q, k, v, _ints(kernel_size), _ints(stride), _ints(dilation),
                                     [bool(c) for c in is_causal], float(scale), _ints(q_tile_shape),
                                     _ints(kv_tile_shape), q_scale, k_scale, v_scale, bool(run_persistent),
                                     bool(anchored_tiles))
    return _lib.fna_forward_fused(q, k, v, kernel_size, stride, dilation, is_causal, scale, q_tile_shape, kv_tile_shape,
                                  q_scale=q_scale, k_scale=k_scale, v_scale=v_scale, run_persistent=run_persistent,
                                  anchored_tiles=anchored_tiles)


def attention_forward(q, k, v, is_causal, scale, q_scale=None, k_scale=None, v_scale=None):
    if _tracing():
        return _attention_forward_op(q, k, v, bool(is_causal), float(scale), q_scale, k_scale, v_scale)
    return _lib.attention_forward(q, k, v, is_causal, scale, q_scale=q_scale, k_scale=k_scale, v_scale=v_scale)


def attention_forward_varlen(q, k, v, cumulative_seqlen_q, cumulative_seqlen_kv, max_seqlen_q, max_seqlen_kv,
                             is_causal, scale, q_scale=None, k_scale=None, v_scale=None):
    if _tracing():
        return _attention_forward_varlen_op(q, k, v, cumulative_seqlen_q, cumulative_seqlen_kv, int(max_seqlen_q),
                                            int(max_seqlen_kv), bool(is_causal), float(scale), q_scale, k_scale,
                                            v_scale)
    return _lib.attention_forward_varlen(q, k, v, cumulative_seqlen_q, cumulative_seqlen_kv, max_seqlen_q,
                                         max_seqlen_kv, is_causal, scale, q_scale=q_scale, k_scale=k_scale,
                                         v_scale=v_scale)


def compute_delta(out, d_out):
    if _tracing():
        return _compute_delta_op(out, d_out)
    return _lib.compute_delta(out, d_out)


def fna_backward(q, k, v, d_out, lse, delta, kernel_size, stride, dilation, is_causal, scale, q_shape, kv_shape,
                 qkv_shape, q_tile_shape, kv_tile_shape):
    if _tracing():
        return _fna_backward_op(q, k, v, d_out, lse, delta, _ints(kernel_size), _ints(stride), _ints(dilation),
                                [bool(c) for c in is_causal], float(scale), _ints(q_shape), _ints(kv_shape),
                                _ints(qkv_shape), _ints(q_tile_shape), _ints(kv_tile_shape))
    return _lib.fna_backward(q, k, v, d_out, lse, delta, kernel_size, stride, dilation, is_causal, scale, q_shape,
                             kv_shape, qkv_shape, q_tile_shape, kv_tile_shape)


def fna_backward_fused(q, k, v, d_out, lse, delta, kernel_size, stride, dilation, is_causal, scale, q_tile_shape,
                       kv_tile_shape, kv_role_q_tile_shape=None, kv_role_kv_tile_shape=None):
    if _tracing():
        return _fna_backward_fused_op(q, k, v, d_out, lse, delta, _ints(kernel_size), _ints(stride), _ints(dilation),
                                      [bool(c) for c in is_causal], float(scale), _ints(q_tile_shape),
                                      _ints(kv_tile_shape),
                                      None if kv_role_q_tile_shape is None else _ints(kv_role_q_tile_shape),
                                      None if kv_role_kv_tile_shape is None else _ints(kv_role_kv_tile_shape))
    return _lib.fna_backward_fused(q, k, v, d_out, lse, delta, kernel_size, stride, dilation, is_causal, scale,
                                   q_tile_shape, kv_tile_shape, kv_role_q_tile_shape, kv_role_kv_tile_shape)


def attention_backward(q, k, v, d_out, lse, delta, seqlen_q, seqlen_kv, is_causal, scale):
    if _tracing():
        return _attention_backward_op(q, k, v, d_out, lse, delta, int(seqlen_q), int(seqlen_kv), bool(is_causal),
                                      float(scale))
    return _lib.attention_backward(q, k, v, d_out, lse, delta, seqlen_q, seqlen_kv, is_causal, scale)


def attention_backward_varlen(q, k, v, d_out, lse, delta, cu_q, cu_kv, padded_cu_q, padded_cu_kv, max_seqlen_q,
                              max_seqlen_kv, is_causal, scale):
    if _tracing():
        return _attention_backward_varlen_op(q, k, v, d_out, lse, delta, cu_q, cu_kv, padded_cu_q, padded_cu_kv,
                                             int(max_seqlen_q), int(max_seqlen_kv), bool(is_causal), float(scale))
    return _lib.attention_backward_varlen(q, k, v, d_out, lse, delta, cu_q, cu_kv, padded_cu_q, padded_cu_kv,
                                          max_seqlen_q, max_seqlen_kv, is_causal, scale)


def token_permute(x, tile_shape, dilation, flip_tiled_dims, widen=False):
    if _tracing():
        return _token_permute_op(x, _ints(tile_shape), _ints(dilation), bool(flip_tiled_dims), bool(widen))
    return _lib.token_permute(x, tile_shape, dilation, flip_tiled_dims, widen=widen)


def token_unpermute(y, token_layout, tile_shape, dilation, flip_tiled_dims):
    if _tracing():
        return _token_unpermute_op(y, _ints(token_layout), _ints(tile_shape), _ints(dilation), bool(flip_tiled_dims))
    return _lib.token_unpermute(y, token_layout, tile_shape, dilation, flip_tiled_dims)


def merge_two(o0, lse0, o1, lse1):
    if _tracing():
        return _merge_two_op(o0, lse0, o1, lse1)
    return _lib.merge_two(o0, lse0, o1, lse1)
