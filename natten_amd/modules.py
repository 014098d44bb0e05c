"""Neighborhood attention layers: QKV projection, na{1,2,3}d, output projection.

Same constructor arguments, parameter names (`qkv`, `proj`) and forward contract as the
reference's src/natten/modules.py:42-132, so its checkpoints load unchanged.  The layers train
(fp16 / bf16): the attention has a backward pass."""

from __future__ import annotations

from typing import Optional

from torch import Tensor, nn

from .checks import check_all_args
from .functional import neighborhood_attention_generic


class NeighborhoodAttentionGeneric(nn.Module):
    def __init__(self, na_dim: int, embed_dim: int, num_heads: int, kernel_size, stride=1, dilation=1,
                 is_causal=False, qkv_bias: bool = True, qk_scale: Optional[float] = None, proj_drop: float = 0.0):
        super().__init__()
        kernel_size, stride, dilation, is_causal = check_all_args(na_dim, kernel_size, stride, dilation, is_causal)
        if embed_dim % num_heads != 0:
            raise ValueError(
                f"Number of attention heads must evenly divide embedding dimension, got {embed_dim=}, {num_heads=}."
            )
        self.na_dim = na_dim
        self.embed_dim = embed_dim
        self.num_heads = num_heads
        self.head_dim = embed_dim // num_heads
        self.scale = qk_scale or self.head_dim**-0.5
        self.kernel_size, self.stride, self.dilation, self.is_causal = kernel_size, stride, dilation, is_causal
        self.qkv = nn.Linear(embed_dim, embed_dim * 3, bias=qkv_bias)
        self.proj = nn.Linear(embed_dim, embed_dim)
        self.proj_drop = nn.Dropout(proj_drop)

    def forward(self, x: Tensor) -> Tensor:
        if x.dim() != self.na_dim + 2:
            raise ValueError(
                f"NeighborhoodAttention{self.na_dim}D expected a tensor with rank {self.na_dim + 2} "
                f"(batch, {self.na_dim} token dimensions, embedding), got {x.dim()=}."
            )
        batch, *tokens, channels = x.shape
        if channels != self.embed_dim:
            raise ValueError(f"Expected embedding dimension {self.embed_dim}, got {channels} ({x.shape=}).")
        # [B, *X, 3, heads, head_dim]: q, k, v are strided views that the operation makes contiguous
        qkv = self.qkv(x).reshape(batch, *tokens, 3, self.num_heads, self.head_dim)
        q, k, v = qkv.unbind(dim=self.na_dim + 1)
        out = neighborhood_attention_generic(
            q, k, v, kernel_size=self.kernel_size, stride=self.stride, dilation=self.dilation,
            is_causal=self.is_causal, scale=self.scale,
        )
        return self.proj_drop(self.proj(out.reshape(batch, *tokens, channels)))

    def extra_repr(self) -> str:
        return (f"head_dim={self.head_dim}, num_heads={self.num_heads}, kernel_size={self.kernel_size}, "
                f"stride={self.stride}, dilation={self.dilation}, is_causal={self.is_causal}")


def _make(na_dim: int):
    class Layer(NeighborhoodAttentionGeneric):
        def __init__(self, embed_dim: int, num_heads: int, kernel_size, stride=1, dilation=1, is_causal=False,
                     qkv_bias: bool = True, qk_scale: Optional[float] = None, proj_drop: float = 0.0):
            super().__init__(na_dim, embed_dim, num_heads, kernel_size, stride, dilation, is_causal, qkv_bias,
                             qk_scale, proj_drop)

    Layer.__name__ = Layer.__qualname__ = f"NeighborhoodAttention{na_dim}D"
    Layer.__doc__ = (f"{na_dim}-D neighborhood attention layer on `[batch, {', '.join('XYZ'[:na_dim])}, embed_dim]` "
                     "inputs: QKV and output projections around the fused attention.")
    return Layer


NeighborhoodAttention1D = _make(1)
NeighborhoodAttention2D = _make(2)
NeighborhoodAttention3D = _make(3)
