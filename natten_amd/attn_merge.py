"""merge_attentions: combine partial attentions over disjoint key sets of the same queries.

Same API and validation as the reference's src/natten/attn_merge.py:193-292; the arithmetic
(:83-95) runs as one HIP kernel per pair.  `torch_compile` is accepted for signature
compatibility and ignored.  With tensors that require grad the merge is an autograd function
that, like the reference's (:130-190), overwrites the partial outputs and LSEs saved by the
originating attention operations with the merged ones and hands every one of them the merged
output's gradient: each attention backward then computes the gradient of attention over the
joint context.  This only works on the tensors those operations returned (or contiguous views of
them), as in the reference."""

from __future__ import annotations

from typing import List, Tuple

import torch
from torch import Tensor

from . import _lib, torch_ops


def merge_attentions(
    outputs: List[Tensor],
    lse_tensors: List[Tensor],
    torch_compile: bool = True,
    use_autograd_fix: bool = True,
) -> Tuple[Tensor, Tensor]:
    if len(outputs) < 2:
        raise ValueError("`merge_attentions` expects at least two tensors.")
    if len(outputs) != len(lse_tensors):
        raise ValueError(
            "`merge_attentions` expected number of outputs and LSE tensors to match, "
            f"got {len(outputs)=} != {len(lse_tensors)}."
        )
    shape = outputs[0].shape
    for i, (output, lse) in enumerate(zip(outputs, lse_tensors)):
        if output.dim() != 4:
            raise ValueError(
                f"Output tensors must be rank-4 tensors with (batch, seq, heads, dim), but got output {i} with "
                f"rank={output.dim()}."
            )
        if output.shape != shape:
            raise ValueError(f"Output tensors must match in shape, but got output {i} with shape={output.shape}.")
        if lse.dim() != 3:
            raise ValueError(
                f"LSE tensors must be rank-3 tensors with (batch, seq, heads), but got LSE {i} with rank={lse.dim()}."
            )
        if lse.shape != shape[:3]:
            raise ValueError(
                f"LSE tensors must match outputs in shape except last dim ({shape=}), but got LSE {i} with "
                f"shape={lse.shape}."
            )
    if torch.is_grad_enabled() and any(t.requires_grad for t in outputs):
        if not use_autograd_fix:
            raise NotImplementedError("natten_amd merges differentiable partial attentions only with use_autograd_fix=True.")
        return MergeAttentionsFunction.apply(*outputs, *lse_tensors)
    return _merge(list(outputs), list(lse_tensors))


def _merge(outputs: List[Tensor], lse_tensors: List[Tensor]) -> Tuple[Tensor, Tensor]:
    out_dtype = outputs[0].dtype
    # more than two partials: keep the running result in float32 between pairwise merges
    work = (lambda t: t.float().contiguous()) if len(outputs) > 2 else (lambda t: t.contiguous())
    out = work(outputs[0])
    lse = lse_tensors[0].float().contiguous()
    for o, l in zip(outputs[1:], lse_tensors[1:]):
        out, lse = torch_ops.merge_two(out, lse, work(o.to(outputs[0].dtype)), l.float().contiguous())
    return out.to(out_dtype), lse


class MergeAttentionsFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, *args):
        n = len(args) // 2
        outputs, lses = args[:n], args[n:]
        with torch.no_grad():
            merged_out, merged_lse = _merge(list(outputs), list(lses))
        ctx.n = n
        ctx.save_for_backward(merged_out, merged_lse, *outputs, *lses)
        return merged_out, merged_lse

    @staticmethod
    def backward(ctx, grad_out, grad_lse):
        n = ctx.n
        merged_out, merged_lse = ctx.saved_tensors[:2]
        outputs = ctx.saved_tensors[2 : 2 + n]
        lses = ctx.saved_tensors[2 + n :]
        for output, lse in zip(outputs, lses):
            output.data.copy_(merged_out.data.reshape(output.shape))
            lse.data.copy_(merged_lse.data.reshape(lse.shape))
        return (grad_out,) * n + (None,) * n


__all__ = ["merge_attentions"]
