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
    scale = scale or head_dim**-0.5
    d_pad = padded_head_dim(head_dim)
    if torch.is_grad_enabled() and (query.requires_grad or key.requires_grad or value.requires_grad):
        if is_fp8(query.dtype):
            raise NotImplementedError("natten_amd attention has no backward pass for 8-bit float operands.")
        if cumulative_seqlen_Q is not None:
            out, lse = AmdFmhaVarlenFunction.apply(
                query, key, value, bool(is_causal), float(scale), cumulative_seqlen_Q, cumulative_seqlen_KV,
                int(max_seqlen_Q), int(max_seqlen_KV),
            )
        else:
            out, lse = AmdFmhaFunction.apply(query, key, value, bool(is_causal), float(scale))
        if out_dtype is not None and out.dtype != out_dtype:
            out = out.to(out_dtype)
        return (out, lse) if return_lse else out
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


def _pad_rows(x: Tensor, rows: int) -> Tensor:
    """Zero-pads dimension 1 to `rows`."""
    if x.shape[1] == rows:
        return x.contiguous()
    pad = [0, 0] * (x.dim() - 2) + [0, rows - x.shape[1]]
    return torch.nn.functional.pad(x, pad).contiguous()


class AmdFmhaFunction(torch.autograd.Function):
    """Dense attention with a backward pass (fp16 / bf16, fixed-length batches): the backward
    kernels of neighborhood attention on the 1-D problem whose window is the whole key sequence,
    sequences zero-padded to multiples of 128 rows.  Counterpart of the reference's
    src/natten/backends/blackwell_fmha.py:52-170; the gradient of LSE is not propagated.  The saved
    output and LSE are the returned tensors themselves (see AmdFnaFunction)."""

    @staticmethod
    def forward(ctx, query, key, value, is_causal, scale):
        with torch.no_grad():
            out, lse = amd_fmha(query, key, value, is_causal=is_causal, scale=scale, return_lse=True)
        ctx.save_for_backward(query, key, value, out, lse)
        ctx.args = (is_causal, scale)
        ctx.mark_non_differentiable(lse)
        return out, lse

    @staticmethod
    def backward(ctx, d_out, d_lse):
        query, key, value, out, lse = ctx.saved_tensors
        is_causal, scale = ctx.args
        head_dim = query.shape[-1]
        d_pad = padded_head_dim(head_dim)
        query, key, value, out, d_out = (
            pad_head_dim(t.contiguous(), d_pad).contiguous() for t in (query, key, value, out, d_out)
        )
        delta = torch_ops.compute_delta(out, d_out)
        sq, skv = query.shape[1], key.shape[1]
        pq, pkv = -(-sq // 128) * 128, -(-skv // 128) * 128
        dq, dk, dv = torch_ops.attention_backward(
            _pad_rows(query, pq), _pad_rows(key, pkv), _pad_rows(value, pkv), _pad_rows(d_out, pq),
            _pad_rows(lse, pq), _pad_rows(delta, pq), sq, skv, is_causal, scale,
        )
        return dq[:, :sq, :, :head_dim], dk[:, :skv, :, :head_dim], dv[:, :skv, :, :head_dim], None, None


class AmdFmhaVarlenFunction(torch.autograd.Function):
    """Variable-length dense attention with a backward pass.  The forward is the sequence-packed
    kernel; the backward runs the fixed-length backward kernels once per sequence (on zero-padded
    copies of its rows), which costs one device-to-host copy of the cumulative lengths and one
    set of launches per sequence.  Counterpart of the varlen arguments of
    src/natten/backends/blackwell_fmha.py:52-170."""

    @staticmethod
    def forward(ctx, query, key, value, is_causal, scale, cu_q, cu_kv, max_q, max_kv):
        with torch.no_grad():
            out, lse = amd_fmha(query, key, value, is_causal=is_causal, scale=scale, return_lse=True,
                                cumulative_seqlen_Q=cu_q, cumulative_seqlen_KV=cu_kv, max_seqlen_Q=max_q,
                                max_seqlen_KV=max_kv)
        ctx.save_for_backward(query, key, value, out, lse, cu_q, cu_kv)
        ctx.args = (is_causal, scale)
        ctx.mark_non_differentiable(lse)
        return out, lse

    @staticmethod
    def backward(ctx, d_out, d_lse):
        query, key, value, out, lse, cu_q, cu_kv = ctx.saved_tensors
        is_causal, scale = ctx.args
        head_dim = query.shape[-1]
        d_pad = padded_head_dim(head_dim)
        q, k, v, o, do = (pad_head_dim(t.contiguous(), d_pad).contiguous() for t in (query, key, value, out, d_out))
        delta = torch_ops.compute_delta(o, do)
        dq, dk, dv = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
        bounds_q, bounds_kv = cu_q.tolist(), cu_kv.tolist()
        for b in range(len(bounds_q) - 1):
            q0, q1, k0, k1 = bounds_q[b], bounds_q[b + 1], bounds_kv[b], bounds_kv[b + 1]
            sq, skv = q1 - q0, k1 - k0
            if sq <= 0 or skv <= 0:
                continue  # no queries, or no keys (output 0, nothing to differentiate)
            pq, pkv = -(-sq // 128) * 128, -(-skv // 128) * 128
            g = torch_ops.attention_backward(
                _pad_rows(q[:, q0:q1], pq), _pad_rows(k[:, k0:k1], pkv), _pad_rows(v[:, k0:k1], pkv),
                _pad_rows(do[:, q0:q1], pq), _pad_rows(lse[:, q0:q1], pq), _pad_rows(delta[:, q0:q1], pq),
                sq, skv, is_causal, scale,
            )
            dq[:, q0:q1] = g[0][:, :sq]
            dk[:, k0:k1] = g[1][:, :skv]
            dv[:, k0:k1] = g[2][:, :skv]
        return (dq[..., :head_dim], dk[..., :head_dim], dv[..., :head_dim]) + (None,) * 6
