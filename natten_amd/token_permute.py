"""Token permute / unpermute front end.

Same contract as the reference's src/natten/token_permute/frontend.py:42-138: returns the
permuted tensor `[B * prod(dilation), prod(ceil(ceil(X/t)/d) * t), H, Dh]` together with the
original token layout and the padded per-dilation-group layout.  The copy itself is the HIP
gather kernel; there is no framework fallback.
"""

from __future__ import annotations

from typing import Optional, Tuple

from torch import Tensor

from . import _lib, torch_ops

DimensionType = Tuple[int, ...]


def _ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


def _check(na_dim: int, tile_shape, dilation):
    if len(tile_shape) != na_dim:
        raise ValueError(f"Expected {na_dim}D tiler for NA{na_dim}D, got {tile_shape=}.")
    if dilation is not None and len(dilation) != na_dim:
        raise ValueError(f"Expected {na_dim}D dilation for NA{na_dim}D, got {dilation=}.")
    if any(int(t) < 1 for t in tile_shape) or (dilation is not None and any(int(d) < 1 for d in dilation)):
        raise ValueError(f"Tile shape and dilation must be positive, got {tile_shape=}, {dilation=}.")


def token_permute_operation(
    tensor: Tensor,
    tile_shape: DimensionType,
    dilation: Optional[DimensionType] = None,
    flip_tiled_dims: bool = True,
    widen: bool = False,
) -> Tuple[Tensor, DimensionType, DimensionType]:
    """`widen=True` (8-bit float input): the permuted tensor holds the same values in bf16."""
    if tensor.dim() not in (4, 5, 6):
        raise ValueError(
            f"Expected 4D, 5D, or 6D tensor (corresponding to NA1D, 2D, 3D), got {tensor.dim()}D input."
        )
    na_dim = tensor.dim() - 3
    _check(na_dim, tile_shape, dilation)
    dilation_ = tuple(int(d) for d in dilation) if dilation is not None else tuple([1] * na_dim)
    tile_shape = tuple(int(t) for t in tile_shape)
    tensor = tensor.contiguous()
    token_layout = tuple(int(x) for x in tensor.shape[1 : 1 + na_dim])
    post = tuple(_ceil_div(_ceil_div(x, t), d) * t for x, t, d in zip(token_layout, tile_shape, dilation_))
    out = torch_ops.token_permute(tensor, tile_shape, dilation_, flip_tiled_dims, widen=widen)
    return out, token_layout, post


def token_unpermute_operation(
    tensor: Tensor,
    token_layout_shape: DimensionType,
    tile_shape: DimensionType,
    dilation: Optional[DimensionType] = None,
    flip_tiled_dims: bool = True,
) -> Tensor:
    if tensor.dim() != 4:
        raise ValueError(f"Expected flattened 4D tensor, got {tensor.dim()}D input.")
    na_dim = len(token_layout_shape)
    _check(na_dim, tile_shape, dilation)
    dilation_ = tuple(int(d) for d in dilation) if dilation is not None else tuple([1] * na_dim)
    groups = 1
    for d in dilation_:
        groups *= d
    if tensor.shape[0] % groups != 0:
        raise ValueError(
            "Expected batch size in token-permuted tensor to be divisible by number of dilation groups "
            f"{groups} ({dilation_=}), got batch={tensor.shape[0]}."
        )
    tensor = tensor.contiguous()
    return torch_ops.token_unpermute(
        tensor, tuple(int(x) for x in token_layout_shape), tuple(int(t) for t in tile_shape), dilation_, flip_tiled_dims
    )
