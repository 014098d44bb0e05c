"""The reference's CPU path for neighborhood attention, restated.  TEST / BENCH INFRASTRUCTURE ONLY
(imported by tests/ and by bench.py's cpu_baseline leg; never by the natten_amd package).

On CPU tensors the reference computes neighborhood attention with one PyTorch call
(src/natten/backends/flex.py:557-709, `flex_fna_generic` without tile shapes):

    block_mask = create_block_mask(mask_mod, B=None, H=None, Q_LEN=N, KV_LEN=N, BLOCK_SIZE=(64, 64), device="cpu")
    out, lse  = flex_attention(q, k, v, block_mask=block_mask, scale=scale, return_lse=True,
                               kernel_options={"FORCE_USE_FLEX_ATTENTION": True}, enable_gqa=...)

on heads-first [B, H, N, D] views of the flattened tokens (flex.py:126-137, :538-547, :645-678), where
`mask_mod` is `single_dim_tiling_mask` (flex.py:333-407): the centre-clamp form of the window test,
evaluated on tensors of flat query / key indices.  `na_mask_mod` below restates that predicate;
tests/test_flex_cpu.py checks it against the oracle's start/end form on every (query, key) pair of
small problems, and the whole call against the dense oracle.

The arithmetic inside `flex_attention` is PyTorch's (torch.nn.attention.flex_attention); this
file only supplies the mask and the layout glue, like the reference does.
"""

from __future__ import annotations

import math
from typing import Sequence, Tuple

import torch


def na_mask_mod(qkv_shape: Sequence[int], kernel_size: Sequence[int], stride: Sequence[int], dilation: Sequence[int],
                is_causal: Sequence[bool]):
    """mask_mod(b, h, q_idx, kv_idx) -> bool tensor: key kv_idx is in the neighborhood of query q_idx
    (row-major flat token indices).  Follows flex.py:333-407 term by term."""
    n = len(qkv_shape)

    def unflatten(idx):
        crd = []
        for X in reversed(qkv_shape):
            crd.append(idx % X)
            idx = idx // X
        return crd[::-1]

    def mask_mod(b, h, q_idx, kv_idx):
        qc, kc = unflatten(q_idx), unflatten(kv_idx)
        ok = None
        for a in range(n):
            X, k, s, d = qkv_shape[a], kernel_size[a], stride[a], dilation[a]
            q_in, k_in = qc[a] // d, kc[a] // d          # coordinates inside the dilation group
            q_grp, k_grp = qc[a] % d, kc[a] % d
            L = (X // d) + 1 - ((q_grp + (d - (X % d))) // d)   # extent of the query's dilation group
            if is_causal[a]:
                leader = torch.minimum((q_in // s) * s + s - 1, L - 1)
                m = (q_in - k_in >= 0) & (leader - k_in < k)
            else:
                left, right = k // 2, k // 2 + (k % 2 - 1)
                leader = torch.minimum((q_in // s) * s + (s // 2), L - 1)
                centre = torch.maximum(torch.minimum(leader, L - 1 - right), left + torch.zeros_like(L))
                w0, w1 = centre - k_in, k_in - centre
                m = ((0 <= w0) & (w0 <= left)) | ((0 <= w1) & (w1 <= right))
            m = m & (q_grp == k_grp)
            ok = m if ok is None else (ok & m)
        return ok

    return mask_mod


def flex_na_cpu(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, kernel_size, stride, dilation, is_causal,
                scale=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Neighborhood attention on heads-last CPU tensors [B, *X, H, D] through the PyTorch call the
    reference's CPU path makes.  Returns (out [B, *X, H, D], lse [B, *X, H])."""
    from torch.nn.attention.flex_attention import create_block_mask, flex_attention

    assert q.device.type == "cpu"
    n = q.dim() - 3
    B, H, D = q.shape[0], q.shape[-2], q.shape[-1]
    Hkv = k.shape[-2]
    shape = tuple(int(x) for x in q.shape[1 : 1 + n])
    N = math.prod(shape)
    scale = scale or D**-0.5
    mask_mod = na_mask_mod(shape, tuple(kernel_size), tuple(stride), tuple(dilation), tuple(bool(c) for c in is_causal))
    block_mask = create_block_mask(mask_mod, B=None, H=None, Q_LEN=N, KV_LEN=N, BLOCK_SIZE=(64, 64), device="cpu")
    q_ = q.reshape(B, N, H, D).transpose(1, 2)
    k_ = k.reshape(B, N, Hkv, D).transpose(1, 2)
    v_ = v.reshape(B, N, Hkv, D).transpose(1, 2)
    out_, lse_ = flex_attention(q_, k_, v_, block_mask=block_mask, scale=scale, return_lse=True,
                                kernel_options={"FORCE_USE_FLEX_ATTENTION": True}, enable_gqa=(H != Hkv))
    out = out_.transpose(1, 2).reshape(B, *shape, H, D)
    lse = lse_.transpose(1, 2).reshape(B, *shape, H)
    return out, lse
