"""Helpers of the GPU parity tests: seeded inputs, oracle calls, tolerances."""

import itertools

import numpy as np
import torch

from oracle import c_oracle
from oracle import na_oracle as O

# Tolerance of the floating-point parity tests for fp16 / bf16 operands: atol = rtol = 1e-2
# against the float64 oracle evaluated on the same (already rounded) inputs.
ATOL = 1e-2
RTOL = 1e-2


def make_qkv(B, shape, H, Hkv, D, dtype, seed=0, std=1.0, device="cuda"):
    gen = torch.Generator().manual_seed(seed)
    q = (torch.randn((B, *shape, H, D), generator=gen) * std).to(dtype)
    k = (torch.randn((B, *shape, Hkv, D), generator=gen) * std).to(dtype)
    v = (torch.randn((B, *shape, Hkv, D), generator=gen) * std).to(dtype)
    return q.to(device), k.to(device), v.to(device)


def to_np(t):
    return t.detach().float().cpu().numpy()


def oracle_full(q, k, v, kernel_size, stride, dilation, is_causal, scale=None):
    return c_oracle.na_forward(to_np(q), to_np(k), to_np(v), kernel_size, stride, dilation, is_causal, scale)


def assert_close(name, got, ref, atol=ATOL, rtol=RTOL):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{name}: non-finite values in result"
    err = np.abs(got - ref)
    bound = atol + rtol * np.abs(ref)
    bad = err > bound
    if bad.any():
        idx = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(
            f"{name}: {int(bad.sum())} of {bad.size} elements out of tolerance; worst at {idx}: "
            f"got {got[idx]:.6f} ref {ref[idx]:.6f} (max abs err {err.max():.3e})"
        )


def tuplify(x, n):
    return tuple([x] * n) if isinstance(x, (int, bool)) else tuple(x)


def stratified_tokens(shape, kernel_size, stride, dilation, is_causal, n_samples, rng):
    """Row-major token indices of `n_samples` query positions chosen to hit every class of window:
    all corners; per dimension the first and last `kernel_size * dilation` coordinates (clamped
    windows of every dilation group at both borders), the first and last coordinates of a causal
    dimension, the coordinates either side of a stride-group boundary; the rest uniform."""
    n = len(shape)
    edge = []
    for X, k, s, d, c in zip(shape, kernel_size, stride, dilation, is_causal):
        w = min(X, k * d)
        e = set(range(w)) | set(range(X - w, X))
        step = s * d
        for b in range(step, X, step):  # last query of a stride group and the first of the next
            e.update(x for x in range(b - d, b + d) if 0 <= x < X)
        edge.append(np.array(sorted(e)))
    coords = [np.array(c) for c in itertools.product(*[(0, X - 1) for X in shape])]
    while len(coords) < n_samples:
        kind = len(coords) % 3
        c = np.empty(n, dtype=np.int64)
        for a in range(n):
            use_edge = kind == 0 or (kind == 1 and rng.integers(0, 2) == 0)
            c[a] = rng.choice(edge[a]) if use_edge else rng.integers(0, shape[a])
        coords.append(c)
    coords = np.stack(coords[:max(n_samples, 1)])
    return np.ravel_multi_index(tuple(coords.T), shape)


def sampled_check(q, k, v, out, lse, kernel, stride, dilation, causal, n_samples, seed, batches=None,
                  atol=ATOL, rtol=RTOL, scale=None, tag=""):
    """Checks `out`, `lse` at a stratified sample of query positions (all heads of each) against the
    C oracle.  `batches`: the batch entries to draw from (each is handed to the oracle on its own,
    so that a many-gigabyte batch never has to exist as float32 on the host)."""
    B = q.shape[0]
    n = q.dim() - 3
    shape = tuple(q.shape[1 : 1 + n])
    N = int(np.prod(shape))
    H, D = q.shape[-2], q.shape[-1]
    kernel, stride, dilation, causal = (tuplify(x, n) for x in (kernel, stride, dilation, causal))
    rng = np.random.default_rng(seed)
    batches = list(range(B)) if batches is None else list(batches)
    per = -(-n_samples // len(batches))
    for b in batches:
        tok = stratified_tokens(shape, kernel, stride, dilation, causal, per, rng)
        bat = np.zeros(len(tok), dtype=np.int32)
        ref_o, ref_l, _ = c_oracle.na_rows(to_np(q[b : b + 1]), to_np(k[b : b + 1]), to_np(v[b : b + 1]), kernel,
                                           stride, dilation, causal, scale, bat, tok, threads=16)
        ti = torch.as_tensor(tok, device=out.device)
        got_o = to_np(out[b].reshape(N, H, out.shape[-1])[ti])
        got_l = to_np(lse[b].reshape(N, H)[ti])
        assert_close(f"sampled out {tag} batch {b}", got_o, ref_o, atol, rtol)
        assert_close(f"sampled lse {tag} batch {b}", got_l, ref_l, atol, rtol)


def routes_agree_bit_for_bit(shape, dilation, kv_tile) -> bool:
    """Whether the one-launch route and the permuted route place every key at the same position of
    its KV tile (then all sums run in the same order and the results are bit-identical).  Not so
    when an extent is no multiple of dilation x KV tile while every dilation group is at least a
    tile wide: the one-launch route then gathers the last tile of such a dimension from one tile
    extent before the group's end (its leading keys masked) instead of padding it."""
    if all(X % (d * t) == 0 for X, d, t in zip(shape, dilation, kv_tile)):
        return True
    return not all(X // d >= t for X, d, t in zip(shape, dilation, kv_tile))


def assert_routes_agree(tag, a, b, shape, dilation, kv_tile) -> bool:
    """Outputs / LSEs of the two routes: bit-equal where the key placement is the same (returns
    True).  Elsewhere they sum in different orders and round their probabilities against different
    stale maxima: two results that each meet the oracle's bar, which is all that is asserted of their
    difference here (returns False: the caller checks each against the oracle)."""
    if routes_agree_bit_for_bit(shape, dilation, kv_tile):
        assert torch.equal(a, b), "the two routes differ: " + tag
        return True
    assert_close("routes " + tag, to_np(a), to_np(b), atol=1e-2, rtol=1e-2)
    return False


def _dim_windows(X, k, s, d, causal):
    """Per token coordinate x of one dimension: (start, end) of its window and its dilation group,
    in token coordinates: x attends y iff y % d == x % d and start[x] <= y // d < end[x]."""
    start = np.empty(X, dtype=np.int64)
    end = np.empty(X, dtype=np.int64)
    for g in range(d):
        L = O.fix_dilation_extent(X, d, g)
        i = np.arange(L)
        st = O.window_start(i, k, s, L, causal)
        start[g::d] = st
        end[g::d] = O.window_end(i, st, k, L, causal)
    return start, end


def sampled_backward_check(q, k, v, d_out, out, lse, dq, dk, dv, kernel, stride, dilation, causal, n_samples, seed,
                           atol, rtol, scale=None, tag=""):
    """Checks gradients at a stratified sample of positions against a float64 evaluation of the
    backward formulas (reference fna_reference_backward.hpp:60-380): dq at sampled queries, dk and dv
    at sampled keys (all heads of each).  The softmax normalisers (`lse`) and `out` (for
    delta = rowsum(dO * O)) are the forward's results, which the forward tests check against the
    oracle on their own; everything else is recomputed from q, k, v, d_out.  One batch entry at a
    time; only the rows a sample needs leave the device."""
    B = q.shape[0]
    n = q.dim() - 3
    shape = tuple(q.shape[1 : 1 + n])
    N = int(np.prod(shape))
    H, Hkv, D = q.shape[-2], k.shape[-2], q.shape[-1]
    r = H // Hkv
    kernel, stride, dilation, causal = (tuplify(x, n) for x in (kernel, stride, dilation, causal))
    scale = float(scale) if scale is not None else float(D) ** -0.5
    wins = [_dim_windows(X, kk, s, d, c) for X, kk, s, d, c in zip(shape, kernel, stride, dilation, causal)]
    rng = np.random.default_rng(seed)
    dev = q.device

    def rows(t, b, tok):  # [len(tok), heads, D] float64
        return t[b].reshape(N, t.shape[-2], -1)[torch.as_tensor(tok, device=dev)].double().cpu().numpy()

    def keys_of(coord):  # tokens attended by the query at `coord`
        per = []
        for a in range(n):
            st, en = wins[a]
            d = dilation[a]
            per.append(np.arange(st[coord[a]], en[coord[a]]) * d + coord[a] % d)
        return np.ravel_multi_index(tuple(m.ravel() for m in np.meshgrid(*per, indexing="ij")), shape)

    def queries_of(coord):  # tokens of the queries that attend the key at `coord`
        per = []
        for a in range(n):
            st, en = wins[a]
            d = dilation[a]
            x = np.arange(coord[a] % d, shape[a], d)
            j = coord[a] // d
            per.append(x[(st[x] <= j) & (j < en[x])])
        return np.ravel_multi_index(tuple(m.ravel() for m in np.meshgrid(*per, indexing="ij")), shape)

    per_batch = -(-n_samples // B)
    for b in range(B):
        toks = stratified_tokens(shape, kernel, stride, dilation, causal, per_batch, rng)
        lse_b = lse[b].reshape(N, H)
        for tok in toks:
            coord = np.unravel_index(int(tok), shape)
            # ---- dq of this query ----------------------------------------------------------------
            ks = keys_of(coord)
            qq, dd, oo = (rows(t, b, [tok])[0] for t in (q, d_out, out))          # [H, D]
            ll = lse_b[int(tok)].double().cpu().numpy()                           # [H]
            kk_, vv_ = rows(k, b, ks), rows(v, b, ks)                             # [W, Hkv, D]
            kk_h, vv_h = np.repeat(kk_, r, axis=1), np.repeat(vv_, r, axis=1)     # [W, H, D]
            p = np.exp(scale * np.einsum("hd,whd->wh", qq, kk_h) - ll[None, :])
            ds = p * (np.einsum("hd,whd->wh", dd, vv_h) - np.sum(dd * oo, axis=-1)[None, :])
            ref_dq = scale * np.einsum("wh,whd->hd", ds, kk_h)
            assert_close(f"sampled dq {tag} batch {b} token {coord}", rows(dq, b, [tok])[0], ref_dq, atol, rtol)
            # ---- dk, dv of the key at the same position --------------------------------------------
            qs = queries_of(coord)
            kx, vx = (rows(t, b, [tok])[0] for t in (k, v))                       # [Hkv, D]
            kx_h, vx_h = np.repeat(kx, r, axis=0), np.repeat(vx, r, axis=0)       # [H, D]
            qa, da, oa = rows(q, b, qs), rows(d_out, b, qs), rows(out, b, qs)     # [Wq, H, D]
            la = lse_b[torch.as_tensor(qs, device=dev)].double().cpu().numpy()    # [Wq, H]
            p = np.exp(scale * np.einsum("whd,hd->wh", qa, kx_h) - la)
            ds = p * (np.einsum("whd,hd->wh", da, vx_h) - np.sum(da * oa, axis=-1))
            ref_dv = np.einsum("wh,whd->hd", p, da).reshape(Hkv, r, D).sum(axis=1)
            ref_dk = scale * np.einsum("wh,whd->hd", ds, qa).reshape(Hkv, r, D).sum(axis=1)
            assert_close(f"sampled dk {tag} batch {b} token {coord}", rows(dk, b, [tok])[0], ref_dk, atol, rtol)
            assert_close(f"sampled dv {tag} batch {b} token {coord}", rows(dv, b, [tok])[0], ref_dv, atol, rtol)
