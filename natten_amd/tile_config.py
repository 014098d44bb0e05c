"""Tile shapes of the MI355X FNA forward kernel.

Plays the role of the reference's per-architecture tables and validators
(src/natten/backends/configs/cutlass_blackwell/__init__.py:44-63, :90-102, :208-256): the
kernel is instantiated for a few (Q tile, KV tile) token counts; a multi-dimensional tile
shape is any factorisation of those counts.  The default picks, per problem, the
factorisation that minimises the (query, key) pairs the kernel visits (padding and partially
masked tiles included), which is separable per dimension and therefore cheap to search.
"""

from __future__ import annotations

import functools
import math
from typing import List, Optional, Tuple

import torch

DimensionType = Tuple[int, ...]

# (Q tile tokens, KV tile tokens) with a kernel instance; first entry = default.
TILE_SIZES: List[Tuple[int, int]] = [(128, 64), (256, 64), (64, 64)]
SUPPORTED_HEAD_DIMS = (32, 64, 128)


def padded_head_dim(head_dim: int) -> int:
    for d in SUPPORTED_HEAD_DIMS:
        if head_dim <= d:
            return d
    raise NotImplementedError(f"natten_amd supports head_dim <= 128, got {head_dim}.")


def _ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


def _win(i: int, k: int, s: int, L: int, causal: bool) -> Tuple[int, int]:
    wl, wr = k // 2, k // 2 + (k % 2 - 1)
    if causal:
        leader = min((i // s) * s + s - 1, L - 1)
        return max(leader - wl - wr, 0), min(i + 1, L)
    leader = min((i // s) * s + s // 2, L - 1)
    st = max(leader - wl, 0) + ((L - wr - leader - 1) if leader + wr >= L else 0)
    return st, st + k


@functools.lru_cache(maxsize=4096)
def _dim_cost(L: int, k: int, s: int, causal: bool, tq: int, tk: int, anchored: bool = False) -> Tuple[int, int]:
    """(visited pairs, fully-unmasked pairs) along one dimension of extent L for Q tile extent tq
    and KV tile extent tk; the totals of a multi-dimensional problem are products of these.
    `anchored`: the KV tiles of a Q tile start at its window's first key (the one-launch forward
    on the original tensors) instead of at multiples of tk."""
    visited = full = 0
    for q0 in range(0, _ceil_div(L, tq) * tq, tq):
        st_f, en_f = _win(q0, k, s, L, causal)
        st_l, en_l = _win(q0 + tq - 1, k, s, L, causal)
        org = st_f if anchored and L >= tk else (st_f // tk) * tk
        n = _ceil_div(en_l - org, tk)
        visited += n * tk * tq
        for t in range(n):
            lo = org + t * tk
            if lo >= st_l and lo + tk <= en_f and lo + tk <= L:
                full += tk * tq
    return visited, full


def visited_pairs(token_layout, kernel_size, stride, dilation, is_causal, q_tile_shape, kv_tile_shape,
                  anchored: bool = True) -> int:
    """(query, key) pairs per head the forward kernel multiplies with these tile shapes: every Q tile
    (padding rows included) times the whole tiles of its KV box, over all dilation groups (counted
    with the extent of the largest group).  `anchored` as in the one-launch forward."""
    total = 1
    for X, k, s, d, c, tq, tk in zip(token_layout, kernel_size, stride, dilation, is_causal, q_tile_shape, kv_tile_shape):
        total *= d * _dim_cost(_ceil_div(int(X), int(d)), int(k), int(s), bool(c), int(tq), int(tk), bool(anchored))[0]
    return total


def _factorisations(total: int, n: int) -> List[DimensionType]:
    if n == 1:
        return [(total,)]
    out = []
    f = 1
    while f <= total:
        if total % f == 0:
            out += [(f,) + rest for rest in _factorisations(total // f, n - 1)]
        f *= 2
    return out


@torch.compiler.assume_constant_result  # (a search over launch constants: not for the tracer to look into)
def choose_tile_shapes(
    token_layout: DimensionType, kernel_size: DimensionType, stride: DimensionType, dilation: DimensionType,
    is_causal: Tuple[bool, ...], q_size: int, kv_size: int, anchored: bool = False,
) -> Tuple[DimensionType, DimensionType]:
    return _choose_tile_shapes(tuple(token_layout), tuple(kernel_size), tuple(stride), tuple(dilation), tuple(is_causal),
                               int(q_size), int(kv_size), bool(anchored))


@functools.lru_cache(maxsize=1024)
def _choose_tile_shapes(
    token_layout: DimensionType, kernel_size: DimensionType, stride: DimensionType, dilation: DimensionType,
    is_causal: Tuple[bool, ...], q_size: int, kv_size: int, anchored: bool = False,
) -> Tuple[DimensionType, DimensionType]:
    n = len(token_layout)
    ext = tuple(_ceil_div(x, d) for x, d in zip(token_layout, dilation))
    best, best_cost = None, None
    for qt in _factorisations(q_size, n):
        for kt in _factorisations(kv_size, n):
            costs = []
            for anch in ((True, False) if anchored else (False,)):
                visited = full = 1
                for a in range(n):
                    v, f = _dim_cost(ext[a], kernel_size[a], stride[a], is_causal[a], qt[a], kt[a], anch)
                    visited *= v
                    full *= f
                costs.append(visited + 0.3 * (visited - full))
            # ties (anchored tiles make many shapes equal): the cost with tiles at multiples of their
            # extent, which is what the token-permuted route pays; then tiles that are long in the
            # last (memory-contiguous) dimensions
            key = (*costs, tuple(-x for x in reversed(qt)), tuple(-x for x in reversed(kt)))
            if best_cost is None or key < best_cost:
                best, best_cost = (qt, kt), key
    assert best is not None
    return best


def check_fna_forward_config(
    input_tensor: torch.Tensor, kernel_size: DimensionType, stride: DimensionType, dilation: DimensionType,
    is_causal: Tuple[bool, ...], q_tile_shape: Optional[DimensionType] = None,
    kv_tile_shape: Optional[DimensionType] = None,
) -> Tuple[DimensionType, DimensionType]:
    """Validate user tile shapes or choose defaults.  Raises ValueError for unsupported shapes."""
    na_dim = input_tensor.dim() - 3
    layout = tuple(int(x) for x in input_tensor.shape[1 : 1 + na_dim])
    if (q_tile_shape is None) != (kv_tile_shape is None):
        raise ValueError("`q_tile_shape` and `kv_tile_shape` must be given together or not at all.")
    if q_tile_shape is None:
        q_size, kv_size = TILE_SIZES[0]
        # the forward runs on the original tensors wherever it can, with KV tiles laid out from each window's first key
        return choose_tile_shapes(layout, tuple(kernel_size), tuple(stride), tuple(dilation), tuple(is_causal), q_size,
                                  kv_size, True)
    from .checks import check_tile_shape

    q_tile_shape = check_tile_shape(q_tile_shape, na_dim, "q_tile_shape")
    kv_tile_shape = check_tile_shape(kv_tile_shape, na_dim, "kv_tile_shape")
    sizes = (math.prod(q_tile_shape), math.prod(kv_tile_shape))
    if sizes not in TILE_SIZES:
        raise ValueError(
            f"Unsupported tile shapes {q_tile_shape=}, {kv_tile_shape=} ({sizes[0]} x {sizes[1]} tokens); "
            f"supported (Q tile, KV tile) token counts are {TILE_SIZES}."
        )
    return q_tile_shape, kv_tile_shape


BACKWARD_TILE_SIZE = 128  # tokens per Q tile and per KV tile of the backward kernels


def check_fna_backward_config(
    input_tensor: torch.Tensor, kernel_size: DimensionType, stride: DimensionType, dilation: DimensionType,
    is_causal: Tuple[bool, ...], q_tile_shape: Optional[DimensionType] = None,
    kv_tile_shape: Optional[DimensionType] = None,
) -> Tuple[DimensionType, DimensionType]:
    """Validate user tile shapes of the backward pass or choose defaults (the role of the reference's
    check_cutlass_blackwell_fna_backward_config, src/natten/backends/configs/checks.py).  Both tiles
    hold 128 tokens; the last extent above 1 must be even (the other role streams half tiles)."""
    na_dim = input_tensor.dim() - 3
    layout = tuple(int(x) for x in input_tensor.shape[1 : 1 + na_dim])
    if (q_tile_shape is None) != (kv_tile_shape is None):
        raise ValueError("`backward_q_tile_shape` and `backward_kv_tile_shape` must be given together or not at all.")
    if q_tile_shape is None:
        return choose_tile_shapes(layout, tuple(kernel_size), tuple(stride), tuple(dilation), tuple(is_causal),
                                  BACKWARD_TILE_SIZE, BACKWARD_TILE_SIZE)
    from .checks import check_tile_shape

    q_tile_shape = check_tile_shape(q_tile_shape, na_dim, "backward_q_tile_shape")
    kv_tile_shape = check_tile_shape(kv_tile_shape, na_dim, "backward_kv_tile_shape")
    for name, t in (("backward_q_tile_shape", q_tile_shape), ("backward_kv_tile_shape", kv_tile_shape)):
        last = [x for x in t if x > 1]
        if math.prod(t) != BACKWARD_TILE_SIZE or not last or last[-1] % 2 != 0:
            raise ValueError(
                f"Unsupported {name}={t}: backward tiles hold {BACKWARD_TILE_SIZE} tokens and their last extent "
                "above 1 must be even."
            )
    return q_tile_shape, kv_tile_shape


def _half_tile(tile: DimensionType) -> DimensionType:
    """The half tile the other role streams: the last extent above 1, halved."""
    t = list(tile)
    t[max(i for i, x in enumerate(t) if x > 1)] //= 2
    return tuple(t)


@torch.compiler.assume_constant_result
def choose_backward_role_tile_shapes(
    token_layout: DimensionType, kernel_size: DimensionType, stride: DimensionType, dilation: DimensionType,
    is_causal: Tuple[bool, ...],
) -> Optional[Tuple[Tuple[DimensionType, DimensionType], Tuple[DimensionType, DimensionType]]]:
    return _choose_backward_role_tile_shapes(tuple(token_layout), tuple(kernel_size), tuple(stride), tuple(dilation),
                                             tuple(is_causal))


@functools.lru_cache(maxsize=1024)
def _choose_backward_role_tile_shapes(
    token_layout: DimensionType, kernel_size: DimensionType, stride: DimensionType, dilation: DimensionType,
    is_causal: Tuple[bool, ...],
) -> Optional[Tuple[Tuple[DimensionType, DimensionType], Tuple[DimensionType, DimensionType]]]:
    """Tile shapes per launch of the backward on the original tensors, where no permuted layout ties
    the two launches together: ((q_tile, kv_tile) of the dq launch, (q_tile, kv_tile) of the dk / dv
    launch).  The dq launch streams half KV tiles past every Q tile, the dk / dv launch half Q tiles
    past every KV tile; each gets the shapes that visit the fewest (query, key) pairs, counted like
    choose_tile_shapes does (partially masked pairs weigh more).  Only shapes that fit every dilation
    group (at least one tile wide in every dimension: what the kernels need on the original tensors)
    qualify; None when there are none."""
    n = len(token_layout)
    shapes = [t for t in _factorisations(BACKWARD_TILE_SIZE, n)
              if all(x // d >= e for x, d, e in zip(token_layout, dilation, t))
              and [e for e in t if e > 1][-1] % 2 == 0]
    if not shapes:
        return None
    ext = tuple(_ceil_div(x, d) for x, d in zip(token_layout, dilation))

    def cost(q_ext: DimensionType, kv_ext: DimensionType) -> float:
        visited = full = 1
        for a in range(n):
            v, f = _dim_cost(ext[a], kernel_size[a], stride[a], is_causal[a], q_ext[a], kv_ext[a])
            visited *= v
            full *= f
        return visited + 0.3 * (visited - full)

    best = []
    for role in (0, 1):
        keyed = []
        for qt in shapes:
            for kt in shapes:
                c = cost(qt, _half_tile(kt)) if role == 0 else cost(_half_tile(qt), kt)
                keyed.append(((c, tuple(-x for x in reversed(qt)), tuple(-x for x in reversed(kt))), (qt, kt)))
        best.append(min(keyed)[1])
    return best[0], best[1]


def get_all_backward_tile_shapes(na_dim: int) -> List[Tuple[DimensionType, DimensionType]]:
    """Every legal (backward_q_tile_shape, backward_kv_tile_shape) of power-of-two extents."""
    shapes = _factorisations(BACKWARD_TILE_SIZE, na_dim)
    return [(qt, kt) for qt in shapes for kt in shapes]


def get_all_tile_shapes(na_dim: int) -> List[Tuple[DimensionType, DimensionType]]:
    """Every legal (q_tile_shape, kv_tile_shape) for an na_dim-dimensional problem."""
    out = []
    for q_size, kv_size in TILE_SIZES:
        for qt in _factorisations(q_size, na_dim):
            for kt in _factorisations(kv_size, na_dim):
                out.append((qt, kt))
    return out
