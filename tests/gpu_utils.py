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


def assert_routes_agree(tag, a, b, shape, dilation, kv_tile):
    """Outputs / LSEs of the two routes: bit-equal where the key placement is the same, else equal up
    to the order of summation (a few units in the last place of the 16-bit result)."""
    if routes_agree_bit_for_bit(shape, dilation, kv_tile):
        assert torch.equal(a, b), "the two routes differ: " + tag
    else:
        assert_close("routes " + tag, to_np(a), to_np(b), atol=4e-3, rtol=8e-3)
