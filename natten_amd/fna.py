"""Driver of the MI355X fused neighborhood attention:
forward = token permute -> fused kernel -> token unpermute (output and LSE), or one launch on
the original tensors; backward = delta, token permutes, the dQ and dK/dV kernels, unpermutes.

Counterpart of the reference's src/natten/backends/blackwell_fna.py:72-318 (autograd function)
and :332-407 (driver).
"""

from __future__ import annotations

from typing import Optional, Tuple, Union

import torch
from torch import Tensor

from . import _lib, torch_ops
from .checks import check_all_args, check_args_against_input, na_tensor_checks
from .tile_config import check_fna_backward_config, check_fna_forward_config, padded_head_dim
from .token_permute import token_permute_operation, token_unpermute_operation

SUPPORTED_DTYPES = (torch.float16, torch.bfloat16, torch.float8_e4m3fn, torch.float8_e5m2)
# neighborhood attention also takes float32 (forward only, token-permuted route, a kernel of its own)
FNA_DTYPES = SUPPORTED_DTYPES + (torch.float32,)
FP8_DTYPES = _lib.FP8_DTYPES


def is_fp8(dtype: torch.dtype) -> bool:
    return dtype in FP8_DTYPES


def resolve_scale(scale, heads: int, device, name: str) -> Optional[Tensor]:
    """Per-head dequantisation scale as a float32 tensor [heads] (or None): accepts None, a
    number, a one-element tensor or a tensor with one entry per head."""
    if scale is None:
        return None
    if not isinstance(scale, Tensor):
        return torch.full((heads,), float(scale), dtype=torch.float32, device=device)
    s = scale.detach().to(device=device, dtype=torch.float32).reshape(-1)
    if s.numel() == 1:
        return s.expand(heads).contiguous()
    if s.numel() != heads:
        raise ValueError(f"{name} must have one entry or one entry per head ({heads}), got {tuple(scale.shape)}.")
    return s.contiguous()


def pad_head_dim(x: Tensor, d_to: int) -> Tensor:
    """Zero-pads the last dimension (8-bit floats through their bytes: 0x00 is +0)."""
    if x.shape[-1] == d_to:
        return x
    if is_fp8(x.dtype):
        return torch.nn.functional.pad(x.view(torch.uint8), (0, d_to - x.shape[-1])).view(x.dtype)
    return torch.nn.functional.pad(x, (0, d_to - x.shape[-1]))


def can_run_amd_fna(query: Tensor, key: Tensor, value: Tensor, raise_error: bool = False) -> bool:
    """MI355X capability check (counterpart of can_run_cutlass_blackwell_fna,
    src/natten/backends/configs/checks.py:143-251)."""

    def no(msg: str, exc=NotImplementedError) -> bool:
        if raise_error:
            raise exc(msg)
        return False

    if not query.is_cuda:
        return no("natten_amd runs on MI355X device tensors only; got a tensor on " + str(query.device) + ".")
    if not _lib.has_lib():
        return no("natten_amd native library is not built (python -m natten_amd.build).", ImportError)
    if query.dtype not in FNA_DTYPES:
        return no(f"natten_amd FNA supports {FNA_DTYPES}, got {query.dtype}.")
    if query.shape[-1] != value.shape[-1]:
        return no("natten_amd FNA does not support different head dims for QK and V.", ValueError)
    if query.shape[-1] > 128 or query.shape[-1] % 8 != 0:
        return no(f"natten_amd FNA supports head_dim <= 128 that is a multiple of 8, got {query.shape[-1]}.")
    if is_fp8(query.dtype) and query.shape[-1] % 16 != 0:
        return no(f"natten_amd FNA needs head dims that are multiples of 16 for 8-bit floats, got {query.shape[-1]}.")
    if is_fp8(query.dtype) and torch.is_grad_enabled() and (query.requires_grad or key.requires_grad or value.requires_grad):
        return no("natten_amd has no backward pass for 8-bit float operands.")
    if query.dtype == torch.float32 and torch.is_grad_enabled() and (query.requires_grad or key.requires_grad or value.requires_grad):
        return no("natten_amd has no backward pass for float32 operands (forward only).")
    return True


_pad_head_dim = pad_head_dim


def _prod(t) -> int:
    out = 1
    for x in t:
        out *= int(x)
    return out


def amd_fna_generic(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    kernel_size,
    stride=1,
    dilation=1,
    is_causal=False,
    scale: Optional[float] = None,
    q_tile_shape=None,
    kv_tile_shape=None,
    return_lse: bool = False,
    q_scale=None,
    k_scale=None,
    v_scale=None,
    out_dtype: Optional[torch.dtype] = None,
    fused: Optional[bool] = None,
    fp8_matmul: Optional[bool] = None,
    backward_q_tile_shape=None,
    backward_kv_tile_shape=None,
    run_persistent_kernel: Optional[bool] = False,
    anchored_tiles: bool = True,
    kv_splits: Optional[int] = None,
    _checked: bool = False,
) -> Union[Tensor, Tuple[Tensor, Tensor]]:
    """`kv_splits` (one-launch path, fp16 / bf16, tiles of 128 x 64 tokens): that many workgroups
    share the KV tiles of every Q tile and their partial results are merged -- for problems with
    fewer Q tiles than the chip has workgroup slots.  None: `functional.kv_splits_default`, unless
    `anchored_tiles` is False or a work-queue launch was asked for (both promise the bits of another
    route); 1: never.  Results differ from the unsplit launch by the rounding of the partial outputs.

    `run_persistent_kernel`: work-queue launch of the forward kernel (resident workgroups pull
    Q tiles from per-XCD queues) instead of a workgroup per Q tile; bit-identical results.  None:
    whichever was measured faster for this kind of problem (`functional.work_queue_default`).

    `anchored_tiles` (one-launch path only): KV tiles are laid out from the first key of a Q tile's
    window instead of from multiples of the tile extent, so that no tile lies partly before the
    window (fewer tiles whenever window starts are not multiples of the tile extent); False keeps
    the permuted path's tiling, and with it bit-identical results to that path.

    `fused` selects the one-launch path that gathers tiles from the original tensors (None:
    whenever the problem allows it); otherwise tokens are permuted, multiplied and unpermuted
    by separate kernels, as the reference does.  Both give bit-identical results.

    8-bit float operands (e4m3fn / e5m2): `q_scale`, `k_scale`, `v_scale` (number or per-head
    tensor) are their dequantisation scales; `out_dtype` defaults to the dtype of `query`, as in
    the reference.  `fp8_matmul` (None: whenever head dim and tiles allow) multiplies them with
    the 8-bit matrix instruction, P rounded to e4m3 as the reference does; False widens them to
    bf16 (exactly) in the token permute and multiplies in bf16, which is slower and more accurate."""
    na_dim = query.dim() - 3
    if not _checked:  # (the public ops have made these checks on the same arguments already)
        na_tensor_checks(query, key, value, must_match_head_dims=True)
        kernel_size, stride, dilation, is_causal = check_all_args(na_dim, kernel_size, stride, dilation, is_causal)
        check_args_against_input(query, kernel_size, stride, dilation, is_causal)
    can_run_amd_fna(query, key, value, raise_error=True)
    q_tile_shape, kv_tile_shape = check_fna_forward_config(
        query, kernel_size, stride, dilation, is_causal, q_tile_shape, kv_tile_shape
    )
    head_dim = query.shape[-1]
    scale = scale or head_dim**-0.5
    d_pad = padded_head_dim(head_dim)
    if run_persistent_kernel is None:
        from .functional import work_queue_default

        run_persistent_kernel = work_queue_default(
            query.shape[0], query.shape[-2], query.shape[1 : 1 + na_dim], kernel_size, stride, dilation, is_causal,
            q_tile_shape, kv_tile_shape)
    if torch.is_grad_enabled() and (query.requires_grad or key.requires_grad or value.requires_grad):
        bwd_q_tile, bwd_kv_tile = check_fna_backward_config(
            query, kernel_size, stride, dilation, is_causal, backward_q_tile_shape, backward_kv_tile_shape
        )
        output, lse = AmdFnaFunction.apply(
            query, key, value, kernel_size, stride, dilation, is_causal, scale, q_tile_shape, kv_tile_shape,
            bwd_q_tile, bwd_kv_tile, fused, bool(run_persistent_kernel), bool(anchored_tiles),
            backward_q_tile_shape is not None,
        )
        if out_dtype is not None and output.dtype != out_dtype:
            output = output.to(out_dtype)
        return (output, lse) if return_lse else output
    if d_pad != head_dim:
        # zero columns change neither q.k nor the first head_dim output columns
        query, key, value = (_pad_head_dim(t, d_pad) for t in (query, key, value))

    in_dtype = query.dtype
    if in_dtype == torch.float32 and not (q_scale is None and k_scale is None and v_scale is None):
        raise ValueError("natten_amd: dequantisation scales belong to 8- and 16-bit operands; float32 operands take none.")
    fp8_ok = (
        is_fp8(in_dtype) and d_pad in (64, 128)
        and _prod(q_tile_shape) == 128 and _prod(kv_tile_shape) == 64
    )
    if fp8_matmul and not fp8_ok:
        raise ValueError(
            "natten_amd: the 8-bit matrix path needs e4m3 / e5m2 operands, head_dim of 64 or 128 (after padding) and "
            f"tiles of 128 x 64 tokens; got {in_dtype}, head_dim {head_dim}, {q_tile_shape=}, {kv_tile_shape=}."
        )
    use_fp8 = fp8_ok and fp8_matmul is not False
    widen = is_fp8(in_dtype) and not use_fp8
    fusable = (not widen) and in_dtype != torch.float32 and _lib.fused_layout_supported(query.shape[1 : 1 + na_dim], dilation, kv_tile_shape,
                                                          row_bytes=key.shape[-2] * d_pad * 2,
                                                          q_tile_shape=q_tile_shape, dtype=in_dtype)
    if fused and not fusable:
        raise ValueError(
            "natten_amd: the fused path needs operands that are not widened and, unless they are fp16 / bf16 with tiles of "
            "128 x 64 tokens, an input extent that is a multiple of "
            f"dilation * KV tile in every dimension; got {tuple(query.shape[1:1 + na_dim])}, {dilation=}, "
            f"{kv_tile_shape=}, {in_dtype}."
        )
    splittable = (
        fusable and fused is not False and in_dtype in (torch.float16, torch.bfloat16)
        and q_scale is None and k_scale is None and v_scale is None
        and _prod(q_tile_shape) == 128 and _prod(kv_tile_shape) == 64 and not torch_ops._tracing()
    )
    if kv_splits is None:
        from .functional import kv_splits_default

        kv_splits = kv_splits_default(
            query.shape[0], query.shape[-2], query.shape[1 : 1 + na_dim], kernel_size, stride, dilation, is_causal,
            q_tile_shape, kv_tile_shape) if (splittable and anchored_tiles and not run_persistent_kernel) else 1
    if not isinstance(kv_splits, int) or not 1 <= kv_splits <= 8:
        raise ValueError(f"natten_amd: kv_splits must be an integer from 1 to 8, got {kv_splits!r}.")
    if kv_splits > 1 and not splittable:
        raise ValueError(
            "natten_amd: kv_splits > 1 needs the one-launch path, fp16 / bf16 operands without dequantisation scales "
            f"and tiles of 128 x 64 tokens (and no graph tracing); got {in_dtype}, {q_tile_shape=}, {kv_tile_shape=}, {fused=}."
        )
    if fusable and fused is not False:
        if kv_splits > 1:
            out_parts, lse_parts = _lib.fna_forward_fused_split(
                query.contiguous(), key.contiguous(), value.contiguous(), kernel_size, stride, dilation, is_causal,
                scale, q_tile_shape, kv_tile_shape, kv_splits, anchored_tiles=bool(anchored_tiles),
            )
            output, lse = _lib.merge_parts(out_parts, lse_parts)
        else:
            output, lse = torch_ops.fna_forward_fused(
                query.contiguous(), key.contiguous(), value.contiguous(), kernel_size, stride, dilation, is_causal,
                scale, q_tile_shape, kv_tile_shape,
                q_scale=resolve_scale(q_scale, query.shape[-2], query.device, "q_scale"),
                k_scale=resolve_scale(k_scale, key.shape[-2], query.device, "k_scale"),
                v_scale=resolve_scale(v_scale, key.shape[-2], query.device, "v_scale"),
                run_persistent=bool(run_persistent_kernel), anchored_tiles=bool(anchored_tiles),
            )
        if d_pad != head_dim:
            output = output[..., :head_dim].contiguous()
        out_dtype = out_dtype or in_dtype
        if output.dtype != out_dtype:
            output = output.to(out_dtype)
        return (output, lse) if return_lse else output

    q_scale = resolve_scale(q_scale, query.shape[-2], query.device, "q_scale")
    k_scale = resolve_scale(k_scale, key.shape[-2], query.device, "k_scale")
    v_scale = resolve_scale(v_scale, key.shape[-2], query.device, "v_scale")

    q_perm, qkv_shape, q_shape = token_permute_operation(query, q_tile_shape, dilation, flip_tiled_dims=True, widen=widen)
    k_perm, _, kv_shape = token_permute_operation(key, kv_tile_shape, dilation, flip_tiled_dims=True, widen=widen)
    v_perm, _, _ = token_permute_operation(value, kv_tile_shape, dilation, flip_tiled_dims=True, widen=widen)

    out_perm, lse_perm = torch_ops.fna_forward(
        q_perm, k_perm, v_perm, kernel_size, stride, dilation, is_causal, scale,
        q_shape, kv_shape, qkv_shape, q_tile_shape, kv_tile_shape,
        q_scale=q_scale, k_scale=k_scale, v_scale=v_scale, run_persistent=bool(run_persistent_kernel),
    )

    output = token_unpermute_operation(out_perm, qkv_shape, q_tile_shape, dilation, flip_tiled_dims=True)
    lse = token_unpermute_operation(
        lse_perm.unsqueeze(-1), qkv_shape, q_tile_shape, dilation, flip_tiled_dims=True
    ).squeeze(-1)
    if d_pad != head_dim:
        output = output[..., :head_dim].contiguous()
    out_dtype = out_dtype or in_dtype
    if output.dtype != out_dtype:
        output = output.to(out_dtype)
    if return_lse:
        return output, lse
    return output


class AmdFnaFunction(torch.autograd.Function):
    """Neighborhood attention with a backward pass (fp16 / bf16, head dims the kernels take).

    Mirrors the reference's autograd function (src/natten/backends/blackwell_fna.py:72-318):
    the forward saves q, k, v, out and LSE; the backward computes delta = rowsum(dO * O), permutes
    q, dO, LSE, delta with the backward Q tile and k, v with the backward KV tile, runs the dQ and
    the dK/dV kernels, and unpermutes the three gradients.  The gradient of the LSE output is
    not propagated, as in the reference.  The saved output and LSE are the returned tensors
    themselves: `merge_attentions` overwrites them with the merged ones before this backward
    runs, which makes it the backward of attention over the joint context."""

    @staticmethod
    def forward(ctx, query, key, value, kernel_size, stride, dilation, is_causal, scale, q_tile_shape, kv_tile_shape,
                bwd_q_tile_shape, bwd_kv_tile_shape, fused, run_persistent_kernel=False, anchored_tiles=True,
                bwd_tiles_given=True):
        with torch.no_grad():
            output, lse = amd_fna_generic(
                query, key, value, kernel_size, stride, dilation, is_causal, scale, q_tile_shape, kv_tile_shape,
                return_lse=True, fused=fused, run_persistent_kernel=run_persistent_kernel,
                anchored_tiles=anchored_tiles,
            )
        ctx.save_for_backward(query, key, value, output, lse)
        ctx.na_args = (kernel_size, stride, dilation, is_causal, scale, bwd_q_tile_shape, bwd_kv_tile_shape)
        ctx.fused = fused
        # the backward may pick tile shapes per launch when the caller fixed none and asked for no
        # other route's bits (anchored_tiles=False promises those of the permuted route)
        ctx.role_tiles = bool(anchored_tiles) and not bwd_tiles_given
        ctx.mark_non_differentiable(lse)
        return output, lse

    @staticmethod
    def backward(ctx, d_output, d_lse):
        query, key, value, output, lse = ctx.saved_tensors
        kernel_size, stride, dilation, is_causal, scale, q_tile, kv_tile = ctx.na_args
        head_dim = query.shape[-1]
        d_pad = padded_head_dim(head_dim)
        # zero columns add nothing to q.k, dO.v or rowsum(dO * O); their gradients are dropped
        query, key, value, output, d_output = (
            pad_head_dim(t.contiguous(), d_pad).contiguous() for t in (query, key, value, output, d_output)
        )
        delta = torch_ops.compute_delta(output, d_output)
        na_dim = len(kernel_size)
        fusable = _lib.backward_fused_layout_supported(query.shape[1 : 1 + na_dim], dilation, q_tile, kv_tile,
                                                       row_bytes=query.shape[-2] * query.shape[-1] * 2)
        if fusable and ctx.fused is not False:
            # the kernels gather and scatter their tiles themselves: no permuted copies; each launch
            # with the tile shapes that visit the fewest tiles for its role
            kv_role = (None, None)
            if ctx.role_tiles:
                from .tile_config import choose_backward_role_tile_shapes

                roles = choose_backward_role_tile_shapes(
                    tuple(int(x) for x in query.shape[1 : 1 + na_dim]), tuple(kernel_size), tuple(stride),
                    tuple(dilation), tuple(is_causal))
                row_bytes = query.shape[-2] * query.shape[-1] * 2
                if roles is not None and all(
                    _lib.backward_fused_layout_supported(query.shape[1 : 1 + na_dim], dilation, qt, kt, row_bytes=row_bytes)
                    for qt, kt in roles
                ):
                    (q_tile, kv_tile), kv_role = roles
            dq, dk, dv = torch_ops.fna_backward_fused(
                query, key, value, d_output, lse.contiguous(), delta, kernel_size, stride, dilation, is_causal, scale,
                q_tile, kv_tile, *kv_role,
            )
            if d_pad != head_dim:
                dq, dk, dv = (t[..., :head_dim].contiguous() for t in (dq, dk, dv))
            return (dq, dk, dv) + (None,) * 13

        def perm(x, tile):
            return token_permute_operation(x.contiguous(), tile, dilation, flip_tiled_dims=True)

        q_perm, qkv_shape, q_shape = perm(query, q_tile)
        do_perm, _, _ = perm(d_output, q_tile)
        lse_perm, _, _ = perm(lse.unsqueeze(-1), q_tile)
        delta_perm, _, _ = perm(delta.unsqueeze(-1), q_tile)
        k_perm, _, kv_shape = perm(key, kv_tile)
        v_perm, _, _ = perm(value, kv_tile)
        dq_perm, dk_perm, dv_perm = torch_ops.fna_backward(
            q_perm, k_perm, v_perm, do_perm, lse_perm.squeeze(-1).contiguous(), delta_perm.squeeze(-1).contiguous(),
            kernel_size, stride, dilation, is_causal, scale, q_shape, kv_shape, qkv_shape, q_tile, kv_tile,
        )
        dq = token_unpermute_operation(dq_perm, qkv_shape, q_tile, dilation, flip_tiled_dims=True)
        dk = token_unpermute_operation(dk_perm, qkv_shape, kv_tile, dilation, flip_tiled_dims=True)
        dv = token_unpermute_operation(dv_perm, qkv_shape, kv_tile, dilation, flip_tiled_dims=True)
        if d_pad != head_dim:
            dq, dk, dv = (t[..., :head_dim].contiguous() for t in (dq, dk, dv))
        return (dq, dk, dv) + (None,) * 13
