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


def _padded_packing(cu: Tensor, rows: int) -> Tuple[Tensor, Tensor, Tensor, int]:
    """A packing of the same sequences with every sequence padded to a multiple of 128 rows, from
    device arithmetic only (no copy to the host): (padded cumulative lengths [sequences + 1] int32,
    padded row of every packed row [rows] int64, which packed rows belong to a sequence [rows]
    bool, row count of the padded packing).  The row count is an upper bound the host can know:
    rows + 127 per sequence, rounded up to 128."""
    num_seqs = cu.numel() - 1
    cu = cu.to(torch.int32)
    padded_len = (cu[1:] - cu[:-1] + 127) // 128 * 128
    padded_cu = torch.cat([cu.new_zeros(1), torch.cumsum(padded_len, 0).to(torch.int32)])
    row = torch.arange(rows, device=cu.device, dtype=torch.int32)
    # the sequence of a packed row (empty sequences own no row; rows past the last sequence belong
    # to none: they count to the last one, which keeps them inside the bound, and their gradients
    # are set to zero afterwards)
    seq = torch.searchsorted(cu[1:].contiguous(), row, right=True).clamp_(max=num_seqs - 1)
    dest = (padded_cu[seq] + (row - cu[seq])).long()
    return padded_cu, dest, row < cu[-1], -(-(rows + 127 * num_seqs) // 128) * 128


def _from_padded_packing(x: Tensor, dest: Tensor, owned: Tensor) -> Tensor:
    """The rows of the packed layout back from the padded packing; rows of no sequence are zero."""
    rows = x.index_select(1, dest)
    return torch.where(owned.view(1, -1, *([1] * (x.dim() - 2))), rows, torch.zeros_like(rows))


def _to_padded_packing(x: Tensor, dest: Tensor, padded_rows: int) -> Tensor:
    out = x.new_zeros((x.shape[0], padded_rows) + tuple(x.shape[2:]))
    return out.index_copy_(1, dest, x)


class AmdFmhaVarlenFunction(torch.autograd.Function):
    """Variable-length dense attention with a backward pass.  The forward is the sequence-packed
    kernel.  The backward kernels work on 128-row tiles that must not straddle two sequences, so
    the backward first copies the operands into a packing whose sequences are padded to multiples
    of 128 rows (index arithmetic on the device, no copy of the lengths to the host), runs one
    set of launches for all sequences, and gathers the gradient rows back.  Counterpart of the
    varlen arguments of src/natten/backends/blackwell_fmha.py:52-170."""

    @staticmethod
    def forward(ctx, query, key, value, is_causal, scale, cu_q, cu_kv, max_q, max_kv):
        with torch.no_grad():
            out, lse = amd_fmha(query, key, value, is_causal=is_causal, scale=scale, return_lse=True,
                                cumulative_seqlen_Q=cu_q, cumulative_seqlen_KV=cu_kv, max_seqlen_Q=max_q,
                                max_seqlen_KV=max_kv)
        ctx.save_for_backward(query, key, value, out, lse, cu_q, cu_kv)
        ctx.args = (is_causal, scale)
        ctx.max_seqlens = (int(max_q), int(max_kv))
        ctx.mark_non_differentiable(lse)
        return out, lse

    @staticmethod
    def backward(ctx, d_out, d_lse):
        query, key, value, out, lse, cu_q, cu_kv = ctx.saved_tensors
        is_causal, scale = ctx.args
        head_dim = query.shape[-1]
        d_pad = padded_head_dim(head_dim)
        q, k, v, o, do = (pad_head_dim(t.contiguous(), d_pad).contiguous() for t in (query, key, value, out, d_out))
        max_q, max_kv = ctx.max_seqlens
        if max_q == 0 or max_kv == 0 or q.shape[1] == 0 or k.shape[1] == 0:
            # no sequence has both queries and keys: the output does not depend on the operands
            return (torch.zeros_like(query), torch.zeros_like(key), torch.zeros_like(value)) + (None,) * 6
        delta = torch_ops.compute_delta(o, do)
        pcu_q, dest_q, owned_q, rows_q = _padded_packing(cu_q, q.shape[1])
        pcu_kv, dest_kv, owned_kv, rows_kv = _padded_packing(cu_kv, k.shape[1])
        dq, dk, dv = torch_ops.attention_backward_varlen(
            _to_padded_packing(q, dest_q, rows_q), _to_padded_packing(k, dest_kv, rows_kv),
            _to_padded_packing(v, dest_kv, rows_kv), _to_padded_packing(do, dest_q, rows_q),
            _to_padded_packing(lse, dest_q, rows_q), _to_padded_packing(delta, dest_q, rows_q),
            cu_q.to(torch.int32).contiguous(), cu_kv.to(torch.int32).contiguous(), pcu_q, pcu_kv, max_q, max_kv,
            is_causal, scale,
        )
        dq = _from_padded_packing(dq, dest_q, owned_q)
        dk, dv = _from_padded_packing(dk, dest_kv, owned_kv), _from_padded_packing(dv, dest_kv, owned_kv)
        return (dq[..., :head_dim], dk[..., :head_dim], dv[..., :head_dim]) + (None,) * 6
