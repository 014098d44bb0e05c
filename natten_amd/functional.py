"""Public operations: attention, na1d, na2d, na3d.

Mirrors the reference's src/natten/functional.py (attention :74-348,
neighborhood_attention_generic :354-564, na1d/na2d/na3d :567-1151): same signatures, same
argument rules and error classes, same self-attention fast path and additional-KV merge.
There is one backend (the MI355X kernels); the reference's NVIDIA-only performance arguments are
accepted and ignored, except `q_tile_shape` / `kv_tile_shape`, which select the kernel's tiles.
"""

from __future__ import annotations

import functools
from typing import Dict, Optional, Tuple, Union

import torch
from torch import Tensor

from .attn_merge import merge_attentions
from .checks import (
    additional_kv_tensor_checks,
    check_all_args,
    check_args_against_input,
    fmha_tensor_checks,
    is_self_attention,
    na_tensor_checks,
)
from .fmha import amd_fmha
from .fna import amd_fna_generic, is_fp8
from .utils.varlen import varlen_tensor_checks

_BACKEND_FNA = "amd-fna"
_BACKEND_FMHA = "amd-fmha"


def attention(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    is_causal: bool = False,
    scale: Optional[float] = None,
    # varlen parameters
    seqlens_Q: Optional[Tensor] = None,
    seqlens_KV: Optional[Tensor] = None,
    cumulative_seqlen_Q: Optional[Tensor] = None,
    cumulative_seqlen_KV: Optional[Tensor] = None,
    max_seqlen_Q: Optional[int] = None,
    max_seqlen_KV: Optional[int] = None,
    # backend parameters
    backend: Optional[str] = None,
    q_tile_size: Optional[int] = None,
    kv_tile_size: Optional[int] = None,
    backward_q_tile_size: Optional[int] = None,
    backward_kv_tile_size: Optional[int] = None,
    backward_kv_splits: Optional[int] = None,
    backward_use_pt_reduction: bool = False,
    run_persistent_kernel: Optional[bool] = None,
    kernel_schedule=None,
    torch_compile: bool = False,
    return_lse: bool = False,
    # quantised (8-bit float) operands; not in the reference
    q_scale=None,
    k_scale=None,
    v_scale=None,
    out_dtype: Optional[torch.dtype] = None,
) -> Union[Tensor, Tuple[Tensor, Tensor]]:
    """Dot product attention on `[batch, seqlen, heads, head_dim]` tensors (heads last).

    `is_causal` is top-left aligned.  Variable-length batches use the sequence-packed layout
    (batch = 1, sequences back to back): pass either `seqlens_Q` / `seqlens_KV` (int32 device
    tensors; costs a synchronisation) or `cumulative_seqlen_{Q,KV}` and `max_seqlen_{Q,KV}` from
    `natten_amd.utils.varlen.generate_varlen_parameters`
    (reference: src/natten/functional.py:74-348).  Returns the output, and the float32 logsumexp
    `[batch, seqlen, heads]` when `return_lse=True`.  For e4m3 / e5m2 operands `q_scale`, `k_scale`,
    `v_scale` (number or per-head tensor) are the dequantisation scales and `out_dtype` the
    result type (default: the operands' type, as in the reference).
    """
    fmha_tensor_checks(query, key, value, must_match_head_dims=True)
    cumulative_seqlen_Q, cumulative_seqlen_KV, max_seqlen_Q, max_seqlen_KV = varlen_tensor_checks(
        query, key, value, seqlens_Q=seqlens_Q, seqlens_KV=seqlens_KV, cumulative_seqlen_Q=cumulative_seqlen_Q,
        cumulative_seqlen_KV=cumulative_seqlen_KV, max_seqlen_Q=max_seqlen_Q, max_seqlen_KV=max_seqlen_KV,
    )
    if backend not in (None, _BACKEND_FMHA):
        raise NotImplementedError(f"Unrecognized attention backend {backend}; natten_amd provides '{_BACKEND_FMHA}'.")
    return amd_fmha(
        query, key, value, is_causal=is_causal, scale=scale, return_lse=return_lse,
        q_scale=q_scale, k_scale=k_scale, v_scale=v_scale, out_dtype=out_dtype,
        cumulative_seqlen_Q=cumulative_seqlen_Q, cumulative_seqlen_KV=cumulative_seqlen_KV,
        max_seqlen_Q=max_seqlen_Q, max_seqlen_KV=max_seqlen_KV,
    )


def neighborhood_attention_generic(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    kernel_size,
    stride=1,
    dilation=1,
    is_causal=False,
    scale: Optional[float] = None,
    additional_keys: Optional[Tensor] = None,
    additional_values: Optional[Tensor] = None,
    attention_kwargs: Optional[Dict] = None,
    # Perf-related args
    backend: Optional[str] = None,
    q_tile_shape=None,
    kv_tile_shape=None,
    backward_q_tile_shape=None,
    backward_kv_tile_shape=None,
    backward_kv_splits=None,
    backward_use_pt_reduction: bool = False,
    run_persistent_kernel: Optional[bool] = None,
    kernel_schedule=None,
    torch_compile: bool = False,
    return_lse: bool = False,
    q_scale=None,
    k_scale=None,
    v_scale=None,
    out_dtype: Optional[torch.dtype] = None,
    fp8_matmul: Optional[bool] = None,
) -> Union[Tensor, Tuple[Tensor, Tensor]]:
    na_tensor_checks(query, key, value)
    additional_kv_tensor_checks(query, key, value, additional_keys, additional_values)
    na_dim = query.dim() - 3
    kernel_size, stride, dilation, is_causal = check_all_args(na_dim, kernel_size, stride, dilation, is_causal)
    check_args_against_input(query, kernel_size=kernel_size, stride=stride, dilation=dilation, is_causal=is_causal)
    if backend not in (None, _BACKEND_FNA):
        raise NotImplementedError(f"Unrecognized backend {backend}; natten_amd provides '{_BACKEND_FNA}'.")

    has_additional_attention = additional_keys is not None and additional_values is not None
    if has_additional_attention and query.dtype == torch.float32:
        # refused before anything is launched: the additional context goes through dense attention
        raise NotImplementedError(
            "natten_amd: float32 operands with additional_keys / additional_values are not supported (dense "
            "attention, which serves the additional context, has no float32 kernel); use fp16 or bf16 operands."
        )
    attn_kwargs = dict(attention_kwargs or {})
    attn_kwargs.pop("torch_compile", None)

    # (float32 operands stay with the neighborhood kernel, which has a float32 form; dense attention has none)
    if query.dtype != torch.float32 and is_self_attention(query, kernel_size=kernel_size, is_causal=is_causal,
                                                          has_additional_attention=has_additional_attention):
        # a window covering the whole input is plain attention over the flattened tokens
        query_shape = query.shape
        q = query.flatten(1, na_dim)
        k = key.flatten(1, na_dim)
        v = value.flatten(1, na_dim)
        if has_additional_attention:
            k = torch.cat([k, additional_keys], dim=1)
            v = torch.cat([v, additional_values], dim=1)
        out, lse = attention(
            q, k, v, is_causal=is_causal[0], scale=scale, return_lse=True,
            q_scale=q_scale, k_scale=k_scale, v_scale=v_scale, out_dtype=out_dtype, **attn_kwargs,
        )
        lse_shape = list(query_shape[:-1])
        out = out.reshape(*lse_shape, v.shape[-1])
        lse = lse.reshape(*lse_shape)
        return (out, lse) if return_lse else out

    scale = scale or query.shape[-1] ** -0.5
    final_dtype = out_dtype or query.dtype
    # Partial results before a merge: bf16 for 8-bit float operands; the operands' own type when
    # gradients are wanted (the merge's backward writes the merged output and LSE into the very
    # tensors the partial attentions saved, so those must reach it uncast); else the final type.
    needs_grad = torch.is_grad_enabled() and any(
        t is not None and t.requires_grad for t in (query, key, value, additional_keys, additional_values)
    )
    if is_fp8(query.dtype):
        work_dtype = torch.bfloat16
    else:
        work_dtype = query.dtype if needs_grad else final_dtype
    output, lse = amd_fna_generic(
        query, key, value, kernel_size=kernel_size, stride=stride, dilation=dilation, is_causal=is_causal,
        scale=scale, q_tile_shape=q_tile_shape, kv_tile_shape=kv_tile_shape, return_lse=True,
        q_scale=q_scale, k_scale=k_scale, v_scale=v_scale,
        out_dtype=work_dtype if has_additional_attention else final_dtype, fp8_matmul=fp8_matmul,
        backward_q_tile_shape=backward_q_tile_shape, backward_kv_tile_shape=backward_kv_tile_shape,
        run_persistent_kernel=run_persistent_kernel, _checked=True,
    )

    if has_additional_attention:
        # the additional keys / values share the dequantisation scales of key / value
        add_out, add_lse = attention(
            query.flatten(1, na_dim), additional_keys, additional_values, is_causal=False, scale=scale,
            return_lse=True, q_scale=q_scale, k_scale=k_scale, v_scale=v_scale, out_dtype=work_dtype, **attn_kwargs,
        )
        merged_out, merged_lse = merge_attentions(
            [output.flatten(1, na_dim), add_out], [lse.flatten(1, na_dim), add_lse]
        )
        output = merged_out.reshape(output.shape).to(final_dtype)
        lse = merged_lse.reshape(output.shape[:-1])

    return (output, lse) if return_lse else output


def _use_work_queue(run_persistent_kernel: Optional[bool], is_causal, num_q_tiles: int = 1 << 30,
                    kv_tiles_per_q_tile: int = 1 << 10) -> bool:
    """`run_persistent_kernel` as given, or the measured default.  The work-queue launch (resident
    workgroups pull Q tiles from per-XCD queues; a workgroup fetches its next position between its last
    KV tile and its stores) saves the 3-4 us a CU slot stands empty between two workgroups of a
    one-workgroup-per-tile launch: 2.5-10 % on the large shapes measured, causal or not; on 2 048 Q
    tiles x 16 KV tiles (c3) the two are within 2 % of each other either way, and below that the queue's
    bookkeeping costs more than it saves.  `num_q_tiles`: Q tiles over all batch entries, dilation
    groups and heads; `kv_tiles_per_q_tile`: KV tiles a Q tile visits (an estimate).  Results are
    bit-identical either way."""
    if run_persistent_kernel is not None:
        return bool(run_persistent_kernel)
    return num_q_tiles >= 2048 and num_q_tiles * kv_tiles_per_q_tile >= 65536


@torch.compiler.assume_constant_result  # (plain Python on launch constants: not for the tracer to look into)
def work_queue_default(batch: int, heads: int, token_layout, kernel_size, stride, dilation, is_causal, q_tile_shape,
                       kv_tile_shape) -> bool:
    """The launch kind the ops pick when `run_persistent_kernel` is None, from the problem's tile counts."""
    return _work_queue_default(int(batch), int(heads), *(tuple(x) for x in (
        token_layout, kernel_size, stride, dilation, is_causal, q_tile_shape, kv_tile_shape)))


@functools.lru_cache(maxsize=1024)
def _work_queue_default(batch, heads, token_layout, kernel_size, stride, dilation, is_causal, q_tile_shape, kv_tile_shape):
    tiles, visits = batch * heads, 1
    for X, k, s, d, qt, kt in zip(token_layout, kernel_size, stride, dilation, q_tile_shape, kv_tile_shape):
        extent = -(-X // d)
        tiles *= -(-extent // qt) * d
        # keys the queries of one Q tile attend along this dimension: a window per stride group the tile spans
        box = min(extent, k + (-(-qt // s) - 1) * s)
        visits *= -(-box // kt)
    return _use_work_queue(None, is_causal, tiles, visits)


@torch.compiler.assume_constant_result
def kv_splits_default(batch: int, heads: int, token_layout, kernel_size, stride, dilation, is_causal, q_tile_shape,
                      kv_tile_shape) -> int:
    """How many workgroups share the KV tiles of a Q tile when `kv_splits` is None: 4 or 2 when the
    problem has so few Q tiles that, split, they still leave every workgroup a compute unit of its
    own (256 of them) and every split has at least four KV tiles of every Q tile; else 1.  Measured
    (split kernel + the 6-7 us merge launch against the unsplit kernel, microseconds): 64 Q tiles of
    34 KV tiles 28 + 6 two ways and 22 + 7 four ways against 46; a 64 x 64 image with 2 heads and a
    33 x 33 window 33 + 6 and 24 + 7 against 58; 256 Q tiles of 34 KV tiles two ways 46 + 6 against
    53 (no gain: the loop only shortens in proportion while a workgroup does not share its SIMDs)."""
    return _kv_splits_default(int(batch), int(heads), *(tuple(x) for x in (
        token_layout, kernel_size, dilation, is_causal, q_tile_shape, kv_tile_shape)))


@functools.lru_cache(maxsize=1024)
def _kv_splits_default(batch, heads, token_layout, kernel_size, dilation, is_causal, q_tile_shape, kv_tile_shape):
    tiles, min_visits = batch * heads, 1
    for X, k, d, c, qt, kt in zip(token_layout, kernel_size, dilation, is_causal, q_tile_shape, kv_tile_shape):
        extent = -(-X // d)
        tiles *= -(-extent // qt) * d
        # fewest KV tiles a Q tile meets along this dimension: a whole window, or one key where causal
        min_visits *= max((1 if c else min(extent, k)) // kt, 1)
    for splits in (4, 2):
        if tiles * splits <= 256 and min_visits >= 4 * splits:
            return splits
    return 1


def _make_na(na_dim: int, name: str):
    def op(
        query: Tensor,
        key: Tensor,
        value: Tensor,
        kernel_size,
        stride=1,
        dilation=1,
        is_causal=False,
        scale: Optional[float] = None,
        additional_keys: Optional[Tensor] = None,
        additional_values: Optional[Tensor] = None,
        attention_kwargs: Optional[Dict] = None,
        backend: Optional[str] = None,
        q_tile_shape=None,
        kv_tile_shape=None,
        backward_q_tile_shape=None,
        backward_kv_tile_shape=None,
        backward_kv_splits=None,
        backward_use_pt_reduction: bool = False,
        run_persistent_kernel: Optional[bool] = None,
        kernel_schedule=None,
        torch_compile: bool = False,
        return_lse: bool = False,
        q_scale=None,
        k_scale=None,
        v_scale=None,
        out_dtype: Optional[torch.dtype] = None,
        fp8_matmul: Optional[bool] = None,
    ) -> Union[Tensor, Tuple[Tensor, Tensor]]:
        if query.dim() != na_dim + 3:
            raise ValueError(
                f"{name} expects rank-{na_dim + 3} tensors [batch, {'*' if na_dim > 1 else ''}tokens, heads, head_dim], "
                f"got rank {query.dim()}."
            )
        return neighborhood_attention_generic(
            query=query, key=key, value=value, kernel_size=kernel_size, stride=stride, dilation=dilation,
            is_causal=is_causal, scale=scale, additional_keys=additional_keys, additional_values=additional_values,
            attention_kwargs=attention_kwargs, backend=backend, q_tile_shape=q_tile_shape,
            kv_tile_shape=kv_tile_shape, backward_q_tile_shape=backward_q_tile_shape,
            backward_kv_tile_shape=backward_kv_tile_shape, backward_kv_splits=backward_kv_splits,
            backward_use_pt_reduction=backward_use_pt_reduction, run_persistent_kernel=run_persistent_kernel,
            kernel_schedule=kernel_schedule, torch_compile=torch_compile, return_lse=return_lse,
            q_scale=q_scale, k_scale=k_scale, v_scale=v_scale, out_dtype=out_dtype, fp8_matmul=fp8_matmul,
        )

    op.__name__ = name
    op.__qualname__ = name
    op.__doc__ = (
        f"{na_dim}-D neighborhood attention on heads-last tensors "
        f"`[batch, {', '.join('XYZ'[:na_dim])}, heads, head_dim]`.\n\n"
        "kernel_size, stride, dilation: int or tuple per dimension (kernel_size >= 2, stride <= kernel_size, "
        "kernel_size * dilation <= input size); is_causal: bool or tuple.  additional_keys / additional_values "
        "`[batch, seqlen, heads_kv, head_dim]` add context every query attends to.  Returns the output and, with "
        "`return_lse=True`, the float32 logsumexp `[batch, *tokens, heads]`.  For e4m3 / e5m2 operands `q_scale`, "
        "`k_scale`, `v_scale` (number or per-head tensor) are the dequantisation scales, `out_dtype` the result "
        "type (default: the operands' type) and `fp8_matmul=False` trades the 8-bit matrix instruction for "
        "bf16 products on exactly widened operands (slower, more accurate)."
    )
    return op


na1d = _make_na(1, "na1d")
na2d = _make_na(2, "na2d")
na3d = _make_na(3, "na3d")

__all__ = ["attention", "na1d", "na2d", "na3d", "neighborhood_attention_generic"]
