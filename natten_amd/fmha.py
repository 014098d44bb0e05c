"""Dense attention forward on MI355X (the callee for additional keys/values and for
kernel_size == input size).  Counterpart of the forward half of the reference's
src/natten/backends/blackwell_fmha.py:190-260, including sequence-packed variable-length batches."""

from __future__ import annotations

from typing import Optional, Tuple, Union

import torch
from torch import Tensor

from . import _lib, torch_ops
from .checks import fmha_tensor_checks
from .fna import SUPPORTED_DTYPES, is_fp8, pad_head_dim, resolve_scale
from .tile_config import padded_head_dim


def amd_fmha(
    query: Tensor, key: Tensor, value: Tensor, is_causal: bool = False, scale: Optional[float] = None,
    return_lse: bool = False,
    q_scale=None,
    k_scale=None,
    v_scale=None,
    out_dtype: Optional[torch.dtype] = None,
    cumulative_seqlen_Q: Optional[Tensor] = None,
    cumulative_seqlen_KV: Optional[Tensor] = None,
    max_seqlen_Q: int = 0,
    max_seqlen_KV: int = 0,
) -> Union[Tensor, Tuple[Tensor, Tensor]]:
    """8-bit float operands are widened to bf16 (exactly) and multiplied in bf16; `q_scale`,
    `k_scale`, `v_scale` (number or per-head tensor) are their dequantisation scales.
    `out_dtype` defaults to the dtype of `query`.  With `cumulative_seqlen_{Q,KV}` (validated by
    the caller) the operands are sequence-packed (batch = 1) and every sequence attends to its
    own keys only."""
    fmha_tensor_checks(query, key, value, must_match_head_dims=True)
    if not query.is_cuda:
        raise NotImplementedError(f"natten_amd runs on MI355X device tensors only; got a tensor on {query.device}.")
    if query.dtype not in SUPPORTED_DTYPES:
        raise NotImplementedError(f"natten_amd attention supports {SUPPORTED_DTYPES}, got {query.dtype}.")
    head_dim = query.shape[-1]
    if head_dim > 128 or head_dim % 8 != 0:
        raise NotImplementedError(f"natten_amd attention supports head_dim <= 128, multiple of 8; got {head_dim}.")
    if is_fp8(query.dtype) and head_dim % 16 != 0:
        raise NotImplementedError(f"natten_amd attention needs head_dim % 16 == 0 for 8-bit floats; got {head_dim}.")
    if torch.is_grad_enabled() and (query.requires_grad or key.requires_grad or value.requires_grad):
        raise NotImplementedError("natten_amd implements the forward pass only; call it under torch.no_grad().")
    scale = scale or head_dim**-0.5
    d_pad = padded_head_dim(head_dim)
    q, k, v = (pad_head_dim(t.contiguous(), d_pad).contiguous() for t in (query, key, value))
    if is_fp8(query.dtype):
        # a one-token tile with no dilation is the identity permutation: a plain widening copy
        q, k, v = (torch_ops.token_permute(t, (1,), (1,), True, widen=True) for t in (q, k, v))
    scales = dict(
        q_scale=resolve_scale(q_scale, q.shape[-2], q.device, "q_scale"),
        k_scale=resolve_scale(k_scale, k.shape[-2], q.device, "k_scale"),
        v_scale=resolve_scale(v_scale, k.shape[-2], q.device, "v_scale"),
    )
    if cumulative_seqlen_Q is not None:
        if max_seqlen_Q == 0 or max_seqlen_KV == 0:
            # every sequence is empty on one side: nothing attends to anything
            out = torch.zeros_like(q)
            lse = torch.full(q.shape[:-1], float("-inf"), dtype=torch.float32, device=q.device)
        else:
            out, lse = torch_ops.attention_forward_varlen(
                q, k, v, cumulative_seqlen_Q.contiguous(), cumulative_seqlen_KV.contiguous(), max_seqlen_Q,
                max_seqlen_KV, bool(is_causal), scale, **scales,
            )
    else:
        out, lse = torch_ops.attention_forward(q, k, v, bool(is_causal), scale, **scales)
    if d_pad != head_dim:
        out = out[..., :head_dim].contiguous()
    out_dtype = out_dtype or query.dtype
    if out.dtype != out_dtype:
        out = out.to(out_dtype)
    if return_lse:
        return out, lse
    return out
