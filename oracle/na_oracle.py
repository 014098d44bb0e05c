"""CPU oracle for neighborhood attention (NA) forward, token permute and attention merge.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this module; it is the
checker that the tests, the smoke entry and the bench's CPU-baseline leg compare the HIP path
against.  Everything is plain numpy (float64 arithmetic for the floating-point parts, exact
integer arithmetic for the index parts).

Each function restates one piece of the reference and cites the file:line it follows
(paths are relative to the SHI-Labs/NATTEN source tree):

  * window interval per dimension ........ csrc/include/natten/cuda/reference/mask.hpp:48-91
  * dilation-group extent ................ csrc/include/natten/cuda/reference/mask.hpp:220-225
  * dense NA mask ........................ csrc/include/natten/cuda/reference/mask.hpp:295-346
  * softmax / LSE convention ............. csrc/include/natten/cuda/reference/fna_reference_forward.hpp:123-208
  * KV tile box of a Q tile .............. csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion.hpp:315-347
  * element mask inside a tile ........... csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion.hpp:384-436
  * token permute / unpermute ............ src/natten/token_permute/torch_impl.py:40-306
  * attention merge ...................... src/natten/attn_merge.py:83-95

Pinning status (what fixes each function without running the reference) is exercised by
tests/test_oracle_*.py: two independent formulations of the window (start/end form here,
centre-clamp form in `window_mask_center_form`, after src/natten/backends/flex.py:360-405),
closed-form invariants, special cases that reduce to plain softmax attention, brute force on
small shapes, and permute round trips against an independent reshape/transpose restatement.
"""

from __future__ import annotations

import itertools
import math
from typing import Optional, Sequence, Tuple

import numpy as np

# ----------------------------------------------------------------------------------------------
# Integer window math
# ----------------------------------------------------------------------------------------------


def window_left(k: int) -> int:
    """mask.hpp:48-51."""
    return k // 2


def window_right(k: int) -> int:
    """mask.hpp:53-57 (k odd: k//2, k even: k//2 - 1)."""
    return k // 2 + (k % 2 - 1)


def window_start(i, k: int, s: int, L: int, causal: bool):
    """First key coordinate attended by query coordinate `i` (scalar or ndarray).

    mask.hpp:59-82.  `L` is the extent of the query's dilation group along this dimension and
    `i` is the coordinate inside that group.
    """
    i = np.asarray(i, dtype=np.int64)
    wl, wr = window_left(k), window_right(k)
    if causal:
        leader = np.minimum((i // s) * s + s - 1, L - 1)
        return np.maximum(leader - wl - wr, 0)
    leader = np.minimum((i // s) * s + s // 2, L - 1)
    return np.maximum(leader - wl, 0) + (leader + wr >= L) * (L - wr - leader - 1)


def window_end(i, start, k: int, L: int, causal: bool):
    """One past the last key coordinate attended (mask.hpp:84-91)."""
    i = np.asarray(i, dtype=np.int64)
    if causal:
        return np.minimum(i + 1, L)
    return np.asarray(start, dtype=np.int64) + k


def fix_dilation_extent(X: int, d: int, g: int) -> int:
    """Number of tokens of dilation group `g` along a dimension of extent X (mask.hpp:220-225)."""
    padding = 1 - ((g + (d - (X % d))) // d)
    return X // d + padding


def _tup(x, n):
    if isinstance(x, (int, bool, np.integer)):
        return tuple([x] * n)
    x = tuple(x)
    assert len(x) == n
    return x


def coords_rowmajor(shape: Sequence[int]) -> np.ndarray:
    """[N, n] integer coordinates of a row-major (torch) token layout."""
    grids = np.meshgrid(*[np.arange(x, dtype=np.int64) for x in shape], indexing="ij")
    return np.stack([g.reshape(-1) for g in grids], axis=-1)


def na_mask_dense(shape, kernel_size, stride=1, dilation=1, is_causal=False) -> np.ndarray:
    """Boolean [N, N] mask, True = query row attends key column.

    Follows NeighborhoodAttentionReferenceMask::apply_mask (mask.hpp:295-346): split each
    global coordinate into (coord // d, coord % d); a pair interacts only inside the same
    dilation group, where the window is evaluated on the group's own extent.
    """
    n = len(shape)
    k, s, d, c = (_tup(kernel_size, n), _tup(stride, n), _tup(dilation, n), _tup(is_causal, n))
    crd = coords_rowmajor(shape)  # [N, n]
    N = crd.shape[0]
    mask = np.ones((N, N), dtype=bool)
    for a in range(n):
        x = crd[:, a]
        xi, xg = x // d[a], x % d[a]
        st = np.empty(N, dtype=np.int64)
        en = np.empty(N, dtype=np.int64)
        for g in range(d[a]):
            sel = xg == g
            Lg = fix_dilation_extent(shape[a], d[a], g)
            st[sel] = window_start(xi[sel], k[a], s[a], Lg, c[a])
            en[sel] = window_end(xi[sel], st[sel], k[a], Lg, c[a])
        m = (xg[:, None] == xg[None, :]) & (xi[None, :] >= st[:, None]) & (xi[None, :] < en[:, None])
        mask &= m
    return mask


def window_mask_center_form(shape, kernel_size, stride=1, dilation=1, is_causal=False) -> np.ndarray:
    """Independent formulation of the same mask (centre-clamp form).

    After single_dim_tiling_mask, src/natten/backends/flex.py:333-407.  Used only to cross-check
    `na_mask_dense`; the two share no code.
    """
    n = len(shape)
    k, s, d, c = (_tup(kernel_size, n), _tup(stride, n), _tup(dilation, n), _tup(is_causal, n))
    crd = coords_rowmajor(shape)
    N = crd.shape[0]
    out = np.ones((N, N), dtype=bool)
    for a in range(n):
        q = crd[:, a][:, None]
        kv = crd[:, a][None, :]
        q_di, kv_di = q // d[a], kv // d[a]
        q_g, kv_g = q % d[a], kv % d[a]
        pad = 1 - ((q_g + (d[a] - (shape[a] % d[a]))) // d[a])
        Lc = shape[a] // d[a] + pad
        wl = k[a] // 2
        wr = k[a] // 2 + (k[a] % 2 - 1)
        if c[a]:
            leader = np.minimum((q_di // s[a]) * s[a] + s[a] - 1, Lc - 1)
            m = (q_di - kv_di >= 0) & (leader - kv_di < k[a]) & (q_g == kv_g)
        else:
            leader = np.minimum((q_di // s[a]) * s[a] + s[a] // 2, Lc - 1)
            center = np.clip(leader, wl, Lc - 1 - wr)
            w0 = center - kv_di
            w1 = kv_di - center
            m = (((0 <= w0) & (w0 <= wl)) | ((0 <= w1) & (w1 <= wr))) & (q_g == kv_g)
        out &= m
    return out


def count_attended(shape, kernel_size, stride=1, dilation=1, is_causal=False) -> int:
    """sum over queries of the number of attended keys (the NA FLOP count's W(q) sum),
    from the closed-form window lengths only (no N x N mask)."""
    n = len(shape)
    k, s, d, c = (_tup(kernel_size, n), _tup(stride, n), _tup(dilation, n), _tup(is_causal, n))
    total = 1
    for a in range(n):
        acc = 0
        for g in range(d[a]):
            Lg = fix_dilation_extent(shape[a], d[a], g)
            i = np.arange(Lg, dtype=np.int64)
            st = window_start(i, k[a], s[a], Lg, c[a])
            en = window_end(i, st, k[a], Lg, c[a])
            acc += int((en - st).sum())
        total *= acc
    return total


# ----------------------------------------------------------------------------------------------
# Dense oracle: O and LSE
# ----------------------------------------------------------------------------------------------


def masked_attention(q, k, v, mask: Optional[np.ndarray], scale: float):
    """softmax(scale * q k^T + mask) v and natural-log LSE of the scaled logits, float64.

    q [B, Nq, H, D], k [B, Nk, Hkv, D], v [B, Nk, Hkv, Dv]; mask [Nq, Nk] bool or None.
    LSE convention: fna_reference_forward.hpp:196-208 (log(sum) + max of *scaled* logits).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    B, Nq, H, D = q.shape
    Hkv = k.shape[2]
    assert H % Hkv == 0
    rep = H // Hkv
    out = np.empty((B, Nq, H, v.shape[-1]), dtype=np.float64)
    lse = np.empty((B, Nq, H), dtype=np.float64)
    for b in range(B):
        for h in range(H):
            hk = h // rep
            s = (q[b, :, h, :] @ k[b, :, hk, :].T) * scale
            if mask is not None:
                s = np.where(mask, s, -np.inf)
            m = s.max(axis=-1, keepdims=True)
            p = np.exp(s - m)
            l = p.sum(axis=-1, keepdims=True)
            out[b, :, h, :] = (p / l) @ v[b, :, hk, :]
            lse[b, :, h] = (np.log(l) + m)[:, 0]
    return out, lse


def na_forward(
    q,
    k,
    v,
    kernel_size,
    stride=1,
    dilation=1,
    is_causal=False,
    scale: Optional[float] = None,
    additional_keys=None,
    additional_values=None,
):
    """Neighborhood attention forward on heads-last tensors [B, *X, H, D] -> (O, LSE).

    With additional keys/values the extra tokens are appended after the self tokens and are
    never masked (mask.hpp:315-322), which is what merge of the two partial attentions computes
    (src/natten/functional.py:524-559).
    """
    q = np.asarray(q)
    shape = q.shape[1:-2]
    n = len(shape)
    B, H, D = q.shape[0], q.shape[-2], q.shape[-1]
    N = int(np.prod(shape))
    scale = float(scale) if scale is not None else float(D) ** -0.5
    mask = na_mask_dense(shape, kernel_size, stride, dilation, is_causal)
    qf = q.reshape(B, N, H, D)
    kf = np.asarray(k).reshape(B, N, k.shape[-2], D)
    vf = np.asarray(v).reshape(B, N, v.shape[-2], v.shape[-1])
    if additional_keys is not None:
        ak = np.asarray(additional_keys)
        av = np.asarray(additional_values)
        kf = np.concatenate([kf, ak], axis=1)
        vf = np.concatenate([vf, av], axis=1)
        mask = np.concatenate([mask, np.ones((N, ak.shape[1]), dtype=bool)], axis=1)
    o, lse = masked_attention(qf, kf, vf, mask, scale)
    return o.reshape(B, *shape, H, vf.shape[-1]), lse.reshape(B, *shape, H)


def masked_attention_backward(q, k, v, d_out, mask: Optional[np.ndarray], scale: float):
    """Gradients of sum(out * d_out) for `masked_attention`, float64, as dense matrix algebra:
    P = softmax(scale q k^T + mask), dV = P^T dO, dP = dO V^T, dS = P * (dP - rowsum(P * dP)),
    dQ = scale dS K, dK = scale dS^T Q  (fna_reference_backward.hpp:116-131, :231-246 evaluate
    the same terms one pair at a time).  The gradient of the LSE output is not propagated."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    d_out = np.asarray(d_out, dtype=np.float64)
    B, Nq, H, D = q.shape
    Hkv = k.shape[2]
    rep = H // Hkv
    dq = np.zeros_like(q)
    dk = np.zeros_like(k)
    dv = np.zeros_like(v)
    for b in range(B):
        for h in range(H):
            hk = h // rep
            s = (q[b, :, h, :] @ k[b, :, hk, :].T) * scale
            if mask is not None:
                s = np.where(mask, s, -np.inf)
            p = np.exp(s - s.max(axis=-1, keepdims=True))
            p /= p.sum(axis=-1, keepdims=True)
            dp = d_out[b, :, h, :] @ v[b, :, hk, :].T
            ds = p * (dp - (p * dp).sum(axis=-1, keepdims=True)) * scale
            dq[b, :, h, :] = ds @ k[b, :, hk, :]
            dk[b, :, hk, :] += ds.T @ q[b, :, h, :]
            dv[b, :, hk, :] += p.T @ d_out[b, :, h, :]
    return dq, dk, dv


def na_backward(q, k, v, d_out, kernel_size, stride=1, dilation=1, is_causal=False, scale: Optional[float] = None):
    """Neighborhood attention backward on heads-last tensors [B, *X, H, D] -> (dQ, dK, dV)."""
    q = np.asarray(q)
    shape = q.shape[1:-2]
    B, H, D = q.shape[0], q.shape[-2], q.shape[-1]
    N = int(np.prod(shape))
    scale = float(scale) if scale is not None else float(D) ** -0.5
    mask = na_mask_dense(shape, kernel_size, stride, dilation, is_causal)
    k = np.asarray(k)
    v = np.asarray(v)
    dq, dk, dv = masked_attention_backward(
        q.reshape(B, N, H, D), k.reshape(B, N, k.shape[-2], D), v.reshape(B, N, v.shape[-2], v.shape[-1]),
        np.asarray(d_out).reshape(B, N, H, v.shape[-1]), mask, scale)
    return dq.reshape(q.shape), dk.reshape(k.shape), dv.reshape(v.shape)


def attention_backward(q, k, v, d_out, is_causal=False, scale: Optional[float] = None):
    """Dense attention backward [B, S, H, D] with optional top-left causal mask -> (dQ, dK, dV)."""
    q = np.asarray(q)
    k = np.asarray(k)
    scale = float(scale) if scale is not None else float(q.shape[-1]) ** -0.5
    mask = None
    if is_causal:
        mask = np.arange(q.shape[1])[:, None] >= np.arange(k.shape[1])[None, :]
    return masked_attention_backward(q, k, v, d_out, mask, scale)


def attention_forward(q, k, v, is_causal=False, scale: Optional[float] = None):
    """Dense attention [B, S, H, D] with optional top-left causal mask -> (O, LSE)."""
    q = np.asarray(q)
    D = q.shape[-1]
    scale = float(scale) if scale is not None else float(D) ** -0.5
    mask = None
    if is_causal:
        Sq, Sk = q.shape[1], np.asarray(k).shape[1]
        mask = np.arange(Sk)[None, :] <= np.arange(Sq)[:, None]
    return masked_attention(q, k, v, mask, scale)


def merge_attentions(outputs, lses):
    """src/natten/attn_merge.py:83-95, float64: pairwise sigmoid / logsigmoid merge."""

    def sigmoid(x):
        return 1.0 / (1.0 + np.exp(-x))

    def logsigmoid(x):
        return -np.logaddexp(0.0, -x)

    outs = [np.asarray(o, dtype=np.float64) for o in outputs]
    ls = [np.asarray(l, dtype=np.float64)[..., None] for l in lses]
    out = outs[0] - sigmoid(ls[1] - ls[0]) * (outs[0] - outs[1])
    lse = ls[0] - logsigmoid(ls[0] - ls[1])
    for i in range(2, len(outs)):
        out = out - sigmoid(ls[i] - lse) * (out - outs[i])
        lse = lse - logsigmoid(lse - ls[i])
    return out, lse[..., 0]


# ----------------------------------------------------------------------------------------------
# Token permute / unpermute (explicit index formula)
# ----------------------------------------------------------------------------------------------


def ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


def permuted_layout(token_layout, tile_shape, dilation):
    """(rest R, padded extent, post-dilation extent) per dimension.

    src/natten/token_permute/torch_impl.py:65-73 (pad to a multiple of tile*dilation) and
    src/natten/token_permute/frontend.py:74 (token_layout_post_dilation).
    """
    R = tuple(ceil_div(ceil_div(x, t), d) for x, t, d in zip(token_layout, tile_shape, dilation))
    padded = tuple(r * t * d for r, t, d in zip(R, tile_shape, dilation))
    post = tuple(r * t for r, t in zip(R, tile_shape))
    return R, padded, post


def permute_source_coords(token_layout, tile_shape, dilation, flip: bool):
    """For every (dilation group g_lin, permuted position p) the source coordinate per dim.

    Returns int64 array [G, S', n]; entries >= token_layout[a] are padding.
    Destination order (torch_impl.py:142-173): [B, delta..., r..., tau..., H, Dh] with the
    per-kind dimension order reversed when `flip` (dim 0 fastest inside each kind), and source
    coordinate x = r*(t*d) + tau*d + delta (view as [R, t, d], torch_impl.py:136-139).
    """
    n = len(token_layout)
    R, _, post = permuted_layout(token_layout, tile_shape, dilation)
    order = list(reversed(range(n))) if flip else list(range(n))
    G = int(np.prod(dilation))
    S = int(np.prod(post))
    out = np.empty((G, S, n), dtype=np.int64)
    d_sizes = [dilation[a] for a in order]
    r_sizes = [R[a] for a in order]
    t_sizes = [tile_shape[a] for a in order]
    g_idx = np.arange(G, dtype=np.int64)
    p_idx = np.arange(S, dtype=np.int64)
    delta = np.unravel_index(g_idx, d_sizes) if G > 0 else []
    rt = np.unravel_index(p_idx, r_sizes + t_sizes)
    for pos, a in enumerate(order):
        dl = np.asarray(delta[pos], dtype=np.int64)[:, None]
        r = np.asarray(rt[pos], dtype=np.int64)[None, :]
        tau = np.asarray(rt[n + pos], dtype=np.int64)[None, :]
        out[:, :, a] = r * (tile_shape[a] * dilation[a]) + tau * dilation[a] + dl
    return out


def token_permute(x: np.ndarray, tile_shape, dilation=None, flip: bool = True):
    """[B, *X, H, Dh] -> ([B*G, S', H, Dh], token_layout, post_dilation_layout); padding = 0."""
    n = x.ndim - 3
    token_layout = tuple(int(v) for v in x.shape[1 : 1 + n])
    dilation = tuple(dilation) if dilation is not None else tuple([1] * n)
    tile_shape = tuple(tile_shape)
    _, _, post = permuted_layout(token_layout, tile_shape, dilation)
    src = permute_source_coords(token_layout, tile_shape, dilation, flip)  # [G, S', n]
    G, S, _ = src.shape
    B, H, Dh = x.shape[0], x.shape[-2], x.shape[-1]
    valid = np.ones((G, S), dtype=bool)
    for a in range(n):
        valid &= src[:, :, a] < token_layout[a]
    lin = np.zeros((G, S), dtype=np.int64)
    for a in range(n):
        lin = lin * token_layout[a] + np.minimum(src[:, :, a], token_layout[a] - 1)
    xf = x.reshape(B, -1, H, Dh)
    out = xf[:, lin.reshape(-1)].reshape(B, G, S, H, Dh).copy()
    out[:, ~valid] = 0
    return out.reshape(B * G, S, H, Dh), token_layout, post


def token_unpermute(y: np.ndarray, token_layout, tile_shape, dilation=None, flip: bool = True):
    """Inverse of token_permute; drops padding.  [B*G, S', H, Dh] -> [B, *X, H, Dh]."""
    n = len(token_layout)
    token_layout = tuple(int(v) for v in token_layout)
    dilation = tuple(dilation) if dilation is not None else tuple([1] * n)
    src = permute_source_coords(token_layout, tuple(tile_shape), dilation, flip)
    G, S, _ = src.shape
    BG, S2, H, Dh = y.shape
    assert S2 == S and BG % G == 0
    B = BG // G
    valid = np.ones((G, S), dtype=bool)
    lin = np.zeros((G, S), dtype=np.int64)
    for a in range(n):
        valid &= src[:, :, a] < token_layout[a]
        lin = lin * token_layout[a] + src[:, :, a]
    N = int(np.prod(token_layout))
    out = np.zeros((B, N, H, Dh), dtype=y.dtype)
    yv = y.reshape(B, G, S, H, Dh)
    out[:, lin[valid]] = yv[:, valid]
    return out.reshape(B, *token_layout, H, Dh)


def token_permute_by_views(x: np.ndarray, tile_shape, dilation=None, flip: bool = True):
    """Independent restatement with pad / reshape / transpose only (no index formula).

    Used in tests to pin `token_permute`; mirrors what a tensor library does with views
    (src/natten/token_permute/torch_impl.py:99-187) rather than computing coordinates.
    """
    n = x.ndim - 3
    layout = x.shape[1 : 1 + n]
    dilation = tuple(dilation) if dilation is not None else tuple([1] * n)
    R, padded, post = permuted_layout(layout, tile_shape, dilation)
    pad = [(0, 0)] + [(0, p - l) for p, l in zip(padded, layout)] + [(0, 0), (0, 0)]
    xp = np.pad(x, pad)
    B, H, Dh = x.shape[0], x.shape[-2], x.shape[-1]
    split = []
    for a in range(n):
        split += [R[a], tile_shape[a], dilation[a]]
    xv = xp.reshape(B, *split, H, Dh)
    dims = list(reversed(range(n))) if flip else list(range(n))
    perm = [0] + [3 * a + 3 for a in dims] + [3 * a + 1 for a in dims] + [3 * a + 2 for a in dims]
    perm += [3 * n + 1, 3 * n + 2]
    xt = np.transpose(xv, perm)
    return np.ascontiguousarray(xt).reshape(B * int(np.prod(dilation)), int(np.prod(post)), H, Dh)


# ----------------------------------------------------------------------------------------------
# Tile-level restatement of the fused kernel's control flow (flat permuted sequences)
# ----------------------------------------------------------------------------------------------


def idx2crd_colex(idx: int, shape: Sequence[int]) -> Tuple[int, ...]:
    """CuTe idx2crd on a compact shape: dimension 0 fastest."""
    out = []
    for s in shape:
        out.append(idx % s)
        idx //= s
    return tuple(out)


def crd2idx_colex(crd: Sequence[int], shape: Sequence[int]) -> int:
    idx, mul = 0, 1
    for c, s in zip(crd, shape):
        idx += c * mul
        mul *= s
    return idx


def kv_tile_box(q_tile_idx, q_shape, q_tile, kv_tile, extent, kernel_size, stride, is_causal):
    """(kv_start coordinate, number of KV tiles) per dim for one Q tile.

    get_trip_count, fna_fusion.hpp:315-347: start from the window start of the tile's first
    query floored to the KV tile, end at the window end of its last query rounded up.
    `extent` is the dilation group's own extent (fna_fusion.hpp:293-311).
    """
    n = len(q_shape)
    q_tiled = tuple(ceil_div(a, b) for a, b in zip(q_shape, q_tile))
    tc = idx2crd_colex(q_tile_idx, q_tiled)
    start, ntiles = [], []
    for a in range(n):
        q_first = tc[a] * q_tile[a]
        q_last = q_first + q_tile[a] - 1
        st_first = int(window_start(q_first, kernel_size[a], stride[a], extent[a], is_causal[a]))
        st_last = int(window_start(q_last, kernel_size[a], stride[a], extent[a], is_causal[a]))
        en_last = int(window_end(q_last, st_last, kernel_size[a], extent[a], is_causal[a]))
        ks = (st_first // kv_tile[a]) * kv_tile[a]
        ke = ceil_div(en_last, kv_tile[a]) * kv_tile[a]
        start.append(ks)
        ntiles.append(ceil_div(ke - ks, kv_tile[a]))
    return tuple(start), tuple(ntiles)


TILE_EMPTY, TILE_PARTIAL, TILE_FULL = 0, 1, 2


def classify_tile(q_first, q_tile, kv_origin, kv_tile, extent, kernel_size, stride, is_causal) -> int:
    """Interval classification of one (Q tile, KV tile) pair.

    FULL  : every key of the KV tile is attended by every query of the Q tile.
    EMPTY : no key of the KV tile is attended by any query of the Q tile.
    Both window start and end are non-decreasing in the query coordinate, so the intersection
    of the windows over the tile is [start(q_last), end(q_first)) and their union is
    [start(q_first), end(q_last)).  (No counterpart in the reference: it decides this once per
    launch, fna_fusion.hpp:503-593; the element mask remains the specification.)
    """
    full, empty = True, False
    for a in range(len(q_tile)):
        qf, ql = q_first[a], q_first[a] + q_tile[a] - 1
        st_f = int(window_start(qf, kernel_size[a], stride[a], extent[a], is_causal[a]))
        en_f = int(window_end(qf, st_f, kernel_size[a], extent[a], is_causal[a]))
        st_l = int(window_start(ql, kernel_size[a], stride[a], extent[a], is_causal[a]))
        en_l = int(window_end(ql, st_l, kernel_size[a], extent[a], is_causal[a]))
        lo, hi = kv_origin[a], kv_origin[a] + kv_tile[a]
        if not (lo >= st_l and hi <= en_f):
            full = False
        if hi <= st_f or lo >= en_l:
            empty = True
    if empty:
        return TILE_EMPTY
    return TILE_FULL if full else TILE_PARTIAL


def fna_forward_tiled(
    q_perm, k_perm, v_perm, kernel_size, stride, dilation, is_causal, scale,
    q_shape, kv_shape, qkv_shape, q_tile, kv_tile, stats: Optional[dict] = None,
):
    """Restates the fused kernel's traversal on token-permuted tensors (flip=True layout).

    q_perm [B*G, SQ', H, D], k_perm/v_perm [B*G, SK', Hkv, D] -> (o_perm, lse_perm), float64.
    For every Q tile: dilation group from the batch index (colexicographic decode,
    fna_fusion.hpp:293-311), KV tile box (`kv_tile_box`), colexicographic tile iteration
    (sm100_fna_load_tma_warpspecialized.hpp:207-229), element mask (fna_fusion.hpp:384-436),
    online softmax over the visited tiles.  EMPTY tiles are skipped, FULL tiles skip the mask.
    """
    n = len(q_shape)
    q_perm = np.asarray(q_perm, dtype=np.float64)
    k_perm = np.asarray(k_perm, dtype=np.float64)
    v_perm = np.asarray(v_perm, dtype=np.float64)
    BG, SQ, H, D = q_perm.shape
    SK, Hkv = k_perm.shape[1], k_perm.shape[2]
    rep = H // Hkv
    G = int(np.prod(dilation))
    qt, kt = int(np.prod(q_tile)), int(np.prod(kv_tile))
    assert SQ % qt == 0 and SK % kt == 0
    q_tiled = tuple(ceil_div(a, b) for a, b in zip(q_shape, q_tile))
    kv_tiled = tuple(ceil_div(a, b) for a, b in zip(kv_shape, kv_tile))
    q_off = np.array([idx2crd_colex(i, q_tile) for i in range(qt)], dtype=np.int64)
    kv_off = np.array([idx2crd_colex(i, kv_tile) for i in range(kt)], dtype=np.int64)
    out = np.zeros((BG, SQ, H, v_perm.shape[-1]), dtype=np.float64)
    lse = np.full((BG, SQ, H), -np.inf, dtype=np.float64)
    counts = {TILE_EMPTY: 0, TILE_PARTIAL: 0, TILE_FULL: 0}
    for bg in range(BG):
        g = idx2crd_colex(bg % G, dilation)
        extent = tuple(fix_dilation_extent(qkv_shape[a], dilation[a], g[a]) for a in range(n))
        for qti in range(SQ // qt):
            tc = idx2crd_colex(qti, q_tiled)
            q_first = tuple(tc[a] * q_tile[a] for a in range(n))
            q_crd = np.array(q_first, dtype=np.int64)[None, :] + q_off  # [qt, n]
            st = np.stack(
                [window_start(q_crd[:, a], kernel_size[a], stride[a], extent[a], is_causal[a]) for a in range(n)], -1
            )
            en = np.stack(
                [window_end(q_crd[:, a], st[:, a], kernel_size[a], extent[a], is_causal[a]) for a in range(n)], -1
            )
            box_start, box_n = kv_tile_box(qti, q_shape, q_tile, kv_tile, extent, kernel_size, stride, is_causal)
            qs = slice(qti * qt, (qti + 1) * qt)
            m_run = np.full((qt, H), -np.inf)
            l_run = np.zeros((qt, H))
            acc = np.zeros((qt, H, v_perm.shape[-1]))
            for it in range(int(np.prod(box_n))):
                itc = idx2crd_colex(it, box_n)
                origin = tuple(box_start[a] + itc[a] * kv_tile[a] for a in range(n))
                cls = classify_tile(q_first, q_tile, origin, kv_tile, extent, kernel_size, stride, is_causal)
                counts[cls] += 1
                if cls == TILE_EMPTY:
                    continue
                kv_lin = crd2idx_colex(tuple(origin[a] // kv_tile[a] for a in range(n)), kv_tiled)
                ks = slice(kv_lin * kt, (kv_lin + 1) * kt)
                kv_crd = np.array(origin, dtype=np.int64)[None, :] + kv_off  # [kt, n]
                if cls == TILE_FULL:
                    msk = np.ones((qt, kt), dtype=bool)
                else:
                    msk = np.ones((qt, kt), dtype=bool)
                    for a in range(n):
                        msk &= (kv_crd[None, :, a] >= st[:, None, a]) & (kv_crd[None, :, a] < en[:, None, a])
                for h in range(H):
                    s = (q_perm[bg, qs, h, :] @ k_perm[bg, ks, h // rep, :].T) * scale
                    s = np.where(msk, s, -np.inf)
                    m_new = np.maximum(m_run[:, h], s.max(axis=-1))
                    m_use = np.where(np.isinf(m_new), 0.0, m_new)
                    alpha = np.exp(m_run[:, h] - m_use)
                    p = np.exp(s - m_use[:, None])
                    l_run[:, h] = l_run[:, h] * alpha + p.sum(axis=-1)
                    acc[:, h, :] = acc[:, h, :] * alpha[:, None] + p @ v_perm[bg, ks, h // rep, :]
                    m_run[:, h] = m_new
            with np.errstate(divide="ignore", invalid="ignore"):
                out[bg, qs] = acc / l_run[:, :, None]
                lse[bg, qs] = np.log(l_run) + m_run
    if stats is not None:
        stats.update({"empty": counts[TILE_EMPTY], "partial": counts[TILE_PARTIAL], "full": counts[TILE_FULL]})
    return out, lse


def na_forward_via_permute(q, k, v, kernel_size, stride, dilation, is_causal, scale, q_tile, kv_tile, stats=None):
    """End-to-end restatement of the token-permute driver
    (src/natten/backends/blackwell_fna.py:108-165): permute -> tiled forward -> unpermute."""
    n = q.ndim - 3
    kernel_size, stride, dilation, is_causal = (
        _tup(kernel_size, n), _tup(stride, n), _tup(dilation, n), _tup(is_causal, n))
    qp, qkv_shape, q_shape = token_permute(np.asarray(q, dtype=np.float64), q_tile, dilation, True)
    kp, _, kv_shape = token_permute(np.asarray(k, dtype=np.float64), kv_tile, dilation, True)
    vp, _, _ = token_permute(np.asarray(v, dtype=np.float64), kv_tile, dilation, True)
    scale = float(scale) if scale is not None else float(q.shape[-1]) ** -0.5
    op, lp = fna_forward_tiled(qp, kp, vp, kernel_size, stride, dilation, is_causal, scale,
                               q_shape, kv_shape, qkv_shape, tuple(q_tile), tuple(kv_tile), stats)
    o = token_unpermute(op, qkv_shape, q_tile, dilation, True)
    l = token_unpermute(lp[..., None], qkv_shape, q_tile, dilation, True)[..., 0]
    return o, l
