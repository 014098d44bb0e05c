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
