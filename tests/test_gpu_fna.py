"""GPU parity: fused neighborhood attention forward through the public API (which goes through
the C ABI), against the CPU oracle on the same seeded inputs.  Tolerance atol = rtol = 1e-2."""

import itertools

import numpy as np
import pytest
import torch

import natten_amd
from natten_amd.fna import amd_fna_generic
from tests import problems
from tests.gpu_utils import assert_close, assert_routes_agree, make_qkv, oracle_full, sampled_check, to_np, tuplify

pytestmark = pytest.mark.gpu

NA = {1: natten_amd.na1d, 2: natten_amd.na2d, 3: natten_amd.na3d}


def run_case(B, H, Hkv, D, shape, k, s, d, causal, dtype, q_tile=None, kv_tile=None, seed=0, std=1.0, samples=None):
    """One problem through the public API against the oracle: every query, or (`samples`) a
    stratified sample of that many query positions where the oracle cannot do all in seconds."""
    n = len(shape)
    k, s, d, causal = (tuplify(x, n) for x in (k, s, d, causal))
    q, kk, v = make_qkv(B, shape, H, Hkv, D, dtype, seed=seed, std=std)
    with torch.no_grad():
        out, lse = NA[n](q, kk, v, k, s, d, causal, q_tile_shape=q_tile, kv_tile_shape=kv_tile, return_lse=True)
    torch.cuda.synchronize()
    assert out.shape == q.shape and out.dtype == dtype
    assert lse.shape == q.shape[:-1] and lse.dtype == torch.float32
    tag = f"{shape} k={k} s={s} d={d} c={causal} {dtype} tiles={q_tile},{kv_tile}"
    if samples is None:
        ref_o, ref_l = oracle_full(q, kk, v, k, s, d, causal)
        assert_close("out " + tag, to_np(out), ref_o)
        assert_close("lse " + tag, to_np(lse), ref_l)
    else:
        assert torch.isfinite(out).all() and torch.isfinite(lse).all(), tag
        sampled_check(q, kk, v, out, lse, k, s, d, causal, samples, seed=seed + 1000, tag=tag)
    if any(kk_ != x for kk_, x in zip(k, shape)) or any(causal):
        # not the dense-attention shortcut: whichever path the call above took (one launch on
        # the original tensors, or permute + kernel + unpermute), the other one must agree: bit for
        # bit wherever both place the keys alike in their tiles
        from natten_amd.tile_config import check_fna_forward_config
        _, kt_used = check_fna_forward_config(q, k, s, d, causal, q_tile, kv_tile)
        # (the call above lays its KV tiles out from the window's first key where it runs on the
        # original tensors; with the permuted path's tiling the same route must give that path's bits)
        with torch.no_grad():
            out1, lse1 = amd_fna_generic(q, kk, v, k, s, d, causal, q_tile_shape=q_tile, kv_tile_shape=kv_tile,
                                         return_lse=True, anchored_tiles=False)
            out2, lse2 = amd_fna_generic(q, kk, v, k, s, d, causal, q_tile_shape=q_tile, kv_tile_shape=kv_tile,
                                         return_lse=True, fused=False)
        exact = assert_routes_agree("output " + tag, out1, out2, shape, d, kt_used)
        assert_routes_agree("LSE " + tag, lse1, lse2, shape, d, kt_used)
        if not exact:
            # the permuted route then stands on its own against the oracle
            if samples is None:
                assert_close("permuted route, output " + tag, to_np(out2), ref_o)
                assert_close("permuted route, LSE " + tag, to_np(lse2), ref_l)
            else:
                sampled_check(q, kk, v, out2, lse2, k, s, d, causal, max(samples // 2, 100), seed=seed + 3000,
                              tag="permuted route, " + tag)
        # the aligned tiling sums in another order than the anchored one above: it meets the same bar
        # against the oracle, not some tighter one against the other route
        if samples is None:
            assert_close("aligned tiles, output " + tag, to_np(out1), ref_o)
            assert_close("aligned tiles, LSE " + tag, to_np(lse1), ref_l)
        else:
            sampled_check(q, kk, v, out1, lse1, k, s, d, causal, max(samples // 2, 100), seed=seed + 2000,
                          tag="aligned tiles, " + tag)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_config1_shape_na1d(dtype):
    # the first benchmark configuration's problem (B=1, heads=2, L=256, D=32, k=7) on the GPU path
    run_case(1, 2, 2, 32, (256,), 7, 1, 1, False, dtype)


@pytest.mark.parametrize("dil", [(1, 1), (2, 2)])
def test_config2_na2d_bf16(dil):
    run_case(2, 8, 8, 64, (64, 64), (13, 13), (1, 1), dil, False, torch.bfloat16)


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_head_dims_and_dtypes_2d(D, dtype):
    run_case(1, 2, 2, D, (20, 24), (5, 7), (2, 1), (1, 2), (False, True), dtype)


@pytest.mark.parametrize("sizes", [(128, 64), (256, 64), (64, 64)])
def test_every_tile_size_3d(sizes):
    qt = {128: (2, 8, 8), 256: (4, 8, 8), 64: (1, 8, 8)}[sizes[0]]
    kt = {64: (1, 8, 8), 128: (2, 8, 8)}[sizes[1]]
    run_case(1, 2, 1, 64, (9, 16, 24), (4, 8, 8), (1, 8, 4), 1, (True, False, False), torch.bfloat16, qt, kt)


def test_reference_1d_problems():
    for i, (B, H, Hkv, D, shape, k, s, d) in enumerate(problems.NA_1D):
        for causal in (False, True):
            run_case(B, H, Hkv, D, shape, k, s, d, (causal,), torch.float16, seed=i)


def test_reference_2d_problems():
    for i, (B, H, Hkv, D, shape, k, s, d) in enumerate(problems.NA_2D):
        for causal in itertools.product([False, True], repeat=2):
            run_case(B, H, Hkv, D, shape, k, s, d, causal, torch.bfloat16, seed=i)


def test_reference_3d_problems():
    for i, (B, H, Hkv, D, shape, k, s, d) in enumerate(problems.NA_3D):
        # above 40 000 tokens the oracle evaluates a stratified sample of the queries instead of all
        samples = 600 if int(np.prod(shape)) > 40000 else None
        for causal in [(False, False, False), (True, False, True), (True, True, True)]:
            run_case(B, H, Hkv, D, shape, k, s, d, causal, torch.bfloat16, seed=i, samples=samples)


def test_reference_1d_long_problems():
    # 32768 tokens, 2048-key windows, strides 1 .. 2048 (the reference's tests/test_blackwell_fna.py:153-176)
    for i, (B, H, Hkv, D, shape, k, s, d) in enumerate(problems.NA_1D_LONG):
        for causal in (False, True):
            run_case(B, H, Hkv, D, shape, k, s, d, (causal,), [torch.bfloat16, torch.float16][i % 2], seed=i,
                     samples=600)


def _random_problem(rng, n):
    """A random legal problem, drawn like the reference's sweep (tests/test_blackwell_fna.py:445-497:
    extents first, then kernel <= extent, stride <= kernel, dilation <= extent // kernel, random
    causal dimensions, batch / heads / KV heads, head dims in multiples of 8) with smaller size limits."""
    max_size = {1: 4096, 2: 72, 3: 26}[n]
    shape = [int(rng.integers(4, max_size + 1)) for _ in range(n)]
    while int(np.prod(shape)) > 20000:
        a = int(rng.integers(0, n))
        shape[a] = max(4, shape[a] // 3)
    tokens = int(np.prod(shape))
    heads = int(rng.integers(1, min(max(1, 4096 // tokens * 4), 4) + 1))
    batch = int(rng.integers(1, min(max(1, (4096 // tokens * 4) // heads), 3) + 1))
    heads_kv = int(rng.choice([h for h in range(1, heads + 1) if heads % h == 0]))
    D = int(rng.choice(np.arange(8, 129, 8)))
    k = tuple(int(rng.integers(2, x + 1)) for x in shape)
    s = tuple(int(rng.integers(1, kk + 1)) for kk in k)
    d = tuple(int(rng.integers(1, x // kk + 1)) for x, kk in zip(shape, k))
    causal = tuple(bool(rng.integers(0, 2)) for _ in range(n))
    return batch, heads, heads_kv, D, tuple(shape), k, s, d, causal


@pytest.mark.parametrize("n", [1, 2, 3])
def test_random_sweep(n):
    # 100 cases per rank (the reference's quick sweeps run 10 per rank, its default budget is 1000)
    rng = np.random.default_rng(2024 + n)
    tiles = natten_amd.get_all_tile_shapes(n)
    for case in range(100):
        B, H, Hkv, D, shape, k, s, d, causal = _random_problem(rng, n)
        dtype = [torch.bfloat16, torch.float16][case % 2]
        # a third of the cases leave the tile shapes to the driver
        qt, kt = tiles[int(rng.integers(0, len(tiles)))] if case % 3 else (None, None)
        # the oracle walks tokens x window keys: sample the queries of the expensive cases
        cost = B * H * int(np.prod(shape)) * int(np.prod(k))
        run_case(B, H, Hkv, D, shape, k, s, d, causal, dtype, qt, kt, seed=case,
                 samples=None if cost < 3e7 else 300)


def test_argument_errors():
    q = torch.randn(1, 16, 16, 2, 32, dtype=torch.bfloat16).cuda()
    with pytest.raises(ValueError):
        natten_amd.na2d(q, q, q, kernel_size=1)
    with pytest.raises(ValueError):
        natten_amd.na2d(q, q, q, kernel_size=(3, 3), stride=(4, 1))
    with pytest.raises(ValueError):
        natten_amd.na2d(q, q, q, kernel_size=(9, 9), dilation=(2, 2))
    with pytest.raises(ValueError):
        natten_amd.na1d(q, q, q, kernel_size=3)
    with pytest.raises(ValueError):
        natten_amd.na2d(q, q, q, kernel_size=3, q_tile_shape=(3, 5), kv_tile_shape=(8, 8))
    with pytest.raises(NotImplementedError):   # float64 has no kernel (float32 has one: tests/test_gpu_fp32.py)
        natten_amd.na2d(q.double(), q.double(), q.double(), kernel_size=3)
    with pytest.raises(NotImplementedError):
        natten_amd.na2d(q.cpu(), q.cpu(), q.cpu(), kernel_size=3)
