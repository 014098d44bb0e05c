"""GPU parity of the one-launch path that gathers tiles from the original tensors
(natten_amd_fna_forward_fused) against the permute + kernel + unpermute path and the oracle."""

import pytest
import torch

import natten_amd
from natten_amd import _lib
from natten_amd.fna import amd_fna_generic
from tests.gpu_utils import (assert_close, assert_routes_agree, make_qkv, oracle_full, routes_agree_bit_for_bit,
                             sampled_check, to_np)

pytestmark = pytest.mark.gpu

CASES = [
    # shape, kernel, stride, dilation, causal, q_tile, kv_tile, heads, heads_kv, D
    ((256,), (9,), (1,), (1,), (True,), (128,), (64,), 2, 1, 64),
    ((384,), (31,), (4,), (2,), (False,), (128,), (64,), 3, 3, 32),
    ((32, 48), (7, 9), (1, 2), (1, 1), (False, True), (8, 16), (8, 8), 4, 2, 64),
    ((32, 32), (5, 5), (1, 1), (2, 2), (False, False), (16, 8), (4, 16), 2, 2, 128),
    # Q tile that does not divide the group extent (padding queries), KV tile that does
    ((24, 40), (6, 8), (2, 3), (1, 1), (True, False), (16, 16), (8, 8), 2, 2, 64),
    ((6, 16, 24), (4, 8, 8), (1, 8, 4), (1, 1, 1), (True, False, False), (2, 8, 8), (1, 8, 8), 2, 1, 64),
    ((8, 16, 16), (3, 5, 4), (1, 2, 1), (2, 1, 2), (False, False, True), (4, 8, 8), (2, 4, 8), 2, 2, 128),
    ((4, 32, 32), (2, 9, 11), (1, 1, 1), (1, 2, 1), (False, False, False), (1, 8, 8), (1, 8, 8), 1, 1, 32),
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_equals_permuted_and_oracle(case, dtype):
    shape, k, s, d, causal, qt, kt, H, Hkv, D = case
    q, kk, v = make_qkv(2, shape, H, Hkv, D, dtype, seed=7)
    assert _lib.fused_layout_supported(shape, d, kt)
    with torch.no_grad():
        out_f, lse_f = amd_fna_generic(q, kk, v, k, s, d, causal, q_tile_shape=qt, kv_tile_shape=kt, return_lse=True,
                                       fused=True, anchored_tiles=False)
        out_p, lse_p = amd_fna_generic(q, kk, v, k, s, d, causal, q_tile_shape=qt, kv_tile_shape=kt, return_lse=True,
                                       fused=False)
        out_a, lse_a = amd_fna_generic(q, kk, v, k, s, d, causal, q_tile_shape=qt, kv_tile_shape=kt, return_lse=True,
                                       fused=True, anchored_tiles=True)
    assert torch.equal(out_f, out_p)
    assert torch.equal(lse_f, lse_p)
    ref_o, ref_l = oracle_full(q, kk, v, k, s, d, causal)
    assert_close("out", to_np(out_f), ref_o)
    assert_close("lse", to_np(lse_f), ref_l)
    # KV tiles laid out from the window's first key: other tiles, same attention
    assert_close("out, anchored tiles", to_np(out_a), ref_o)
    assert_close("lse, anchored tiles", to_np(lse_a), ref_l)


def test_fused_rejects_what_no_kernel_instance_gathers():
    # a dilation group narrower than the KV tile needs the instance that clamps its gathers, which
    # exists for tiles of 128 x 64 tokens: other tile pairs take the permuted route
    q, kk, v = make_qkv(1, (20, 6), 2, 2, 64, torch.bfloat16, seed=1)
    args = ((5, 3), (1, 1), (1, 1), (False, False))
    assert not _lib.fused_layout_supported((20, 6), (1, 1), (8, 8))
    assert not _lib.fused_layout_supported((20, 6), (1, 1), (8, 8), q_tile_shape=(8, 8), dtype=torch.bfloat16)
    assert _lib.fused_layout_supported((20, 6), (1, 1), (8, 8), q_tile_shape=(16, 8), dtype=torch.bfloat16)
    assert _lib.fused_layout_supported((20, 24), (1, 1), (8, 8), q_tile_shape=(8, 8), dtype=torch.bfloat16)
    # 8-bit operands: taken while every dilation group is at least a KV tile wide, never by the clamping instance
    assert _lib.fused_layout_supported((20, 24), (1, 1), (8, 8), q_tile_shape=(8, 8), dtype=torch.float8_e4m3fn)
    assert not _lib.fused_layout_supported((20, 6), (1, 1), (8, 8), q_tile_shape=(16, 8), dtype=torch.float8_e4m3fn)
    with pytest.raises(ValueError):
        amd_fna_generic(q, kk, v, *args, q_tile_shape=(8, 8), kv_tile_shape=(8, 8), fused=True)
    with pytest.raises(RuntimeError):
        _lib.fna_forward_fused(q, kk, v, *args, 0.125, (8, 8), (8, 8))
    # the default picks the permuted path there and still matches the oracle
    with torch.no_grad():
        out, lse = natten_amd.na2d(q, kk, v, *args, q_tile_shape=(8, 8), kv_tile_shape=(8, 8), return_lse=True)
    ref_o, ref_l = oracle_full(q, kk, v, *args)
    assert_close("out", to_np(out), ref_o)
    assert_close("lse", to_np(lse), ref_l)


EDGE_CASES = [
    # shape, kernel, stride, dilation, heads, heads_kv, D, q_tile, kv_tile: extents that are not
    # multiples of dilation x KV tile (the reference's odd-sized problems among them)
    ((125,), (15,), (1,), (1,), 2, 2, 64, (128,), (64,)),
    ((125,), (3,), (1,), (1,), 1, 1, 32, (128,), (64,)),
    ((257,), (8,), (7,), (5,), 2, 1, 64, (128,), (64,)),
    ((84, 19), (7, 3), (1, 1), (1, 1), 1, 1, 32, (16, 8), (8, 8)),
    ((84, 19), (7, 3), (1, 1), (5, 1), 1, 1, 32, (16, 8), (8, 8)),
    ((19, 29), (8, 8), (1, 1), (2, 3), 1, 1, 128, (8, 16), (8, 8)),
    ((67, 80), (12, 7), (8, 4), (5, 11), 1, 1, 128, (16, 8), (4, 16)),
    ((5, 25), (5, 16), (1, 16), (1, 1), 2, 1, 48, (4, 32), (4, 16)),
    ((33, 33), (24, 16), (1, 1), (1, 1), 1, 1, 128, (8, 16), (8, 8)),
    ((13, 11, 9), (3, 4, 3), (2, 3, 3), (3, 2, 2), 1, 1, 32, (2, 8, 8), (1, 8, 8)),
    ((18, 37, 12), (14, 16, 12), (12, 8, 1), (1, 2, 1), 1, 1, 64, (4, 8, 4), (2, 8, 4)),
    ((57, 20, 88), (20, 4, 6), (1, 1, 1), (2, 1, 1), 1, 1, 72, (2, 4, 16), (2, 4, 8)),
    # the other tile sizes (every group at least a tile wide)
    ((84, 19), (7, 3), (1, 1), (1, 1), 2, 1, 64, (8, 8), (8, 8)),
    ((30, 27, 21), (5, 9, 7), (1, 3, 1), (2, 1, 1), 1, 1, 128, (4, 8, 8), (1, 8, 8)),
]


@pytest.mark.parametrize("case", EDGE_CASES)
def test_fused_on_extents_that_tiles_do_not_divide(case):
    # one launch on the original tensors whatever the extents, within tolerance of the oracle,
    # non-causal and causal.  Where a dilation group is narrower than the KV tile the kernel clamps
    # its gathers, every key keeps its place in the tile and the result is bit-equal to permute +
    # kernel + unpermute; elsewhere the last tile of a dimension is gathered from one tile extent
    # before the group's end and the two routes agree up to the order of summation
    shape, k, s, d, H, Hkv, D, qt, kt = case
    n = len(shape)
    assert not all(X % (dd * t) == 0 for X, dd, t in zip(shape, d, kt))
    for ci, causal in enumerate([(False,) * n, (True,) + (False,) * (n - 1), (True,) * n]):
        dtype = [torch.bfloat16, torch.float16][ci % 2]
        q, kk, v = make_qkv(2, shape, H, Hkv, D, dtype, seed=13 + ci)
        with torch.no_grad():
            out_f, lse_f = amd_fna_generic(q, kk, v, k, s, d, causal, q_tile_shape=qt, kv_tile_shape=kt,
                                           return_lse=True, fused=True, anchored_tiles=False)
            out_p, lse_p = amd_fna_generic(q, kk, v, k, s, d, causal, q_tile_shape=qt, kv_tile_shape=kt,
                                           return_lse=True, fused=False)
            out_a, lse_a = amd_fna_generic(q, kk, v, k, s, d, causal, q_tile_shape=qt, kv_tile_shape=kt,
                                           return_lse=True, fused=True, anchored_tiles=True)
        tag = f"{shape} k={k} s={s} d={d} c={causal}"
        exact = assert_routes_agree("output " + tag, out_f, out_p, shape, d, kt)
        assert_routes_agree("LSE " + tag, lse_f, lse_p, shape, d, kt)
        # both tilings of the one-launch route against the oracle (they sum in different orders: each
        # meets the oracle's bar, not some tighter one against the other), and the permuted route
        # too where it is not bit-equal to the aligned tiling
        routes = [("aligned tiles", out_f, lse_f), ("anchored tiles", out_a, lse_a)]
        if not exact:
            routes.append(("permuted route", out_p, lse_p))
        for name, o, l in routes:
            if int(torch.tensor(shape).prod()) <= 40000:
                ref_o, ref_l = oracle_full(q, kk, v, k, s, d, causal)
                assert_close(f"{name}, out {tag}", to_np(o), ref_o)
                assert_close(f"{name}, lse {tag}", to_np(l), ref_l)
            else:
                sampled_check(q, kk, v, o, l, k, s, d, causal, 400, seed=ci, tag=f"{name}, {tag}")


def test_fused_with_dequantisation_scales():
    q, kk, v = make_qkv(1, (16, 16), 4, 2, 64, torch.bfloat16, seed=3)
    sq = torch.tensor([0.5, 1.0, 2.0, 0.25], device="cuda")
    sk = torch.tensor([1.5, 0.75], device="cuda")
    sv = torch.tensor([2.0, 0.5], device="cuda")
    args = ((5, 5), (1, 1), (1, 1), (False, False))
    with torch.no_grad():
        out_f, lse_f = amd_fna_generic(q, kk, v, *args, return_lse=True, q_scale=sq, k_scale=sk, v_scale=sv, fused=True,
                                       anchored_tiles=False)
        out_p, lse_p = amd_fna_generic(q, kk, v, *args, return_lse=True, q_scale=sq, k_scale=sk, v_scale=sv, fused=False)
    assert torch.equal(out_f, out_p) and torch.equal(lse_f, lse_p)
    qd = q.float() * sq.view(1, 1, 1, -1, 1)
    kd = kk.float() * sk.view(1, 1, 1, -1, 1)
    vd = v.float() * sv.view(1, 1, 1, -1, 1)
    ref_o, ref_l = oracle_full(qd, kd, vd, *args)
    assert_close("out", to_np(out_f), ref_o, atol=2e-2, rtol=1e-2)
    assert_close("lse", to_np(lse_f), ref_l)


# ---- work-queue launch (run_persistent_kernel) ------------------------------------------------------

QUEUE_CASES = [
    # shape, kernel, stride, dilation, causal, heads, heads_kv, D  (default 128 x 64 token tiles)
    ((2000,), (65,), (8,), (3,), (True,), 2, 1, 64),
    ((40, 48), (9, 11), (2, 1), (1, 2), (False, False), 4, 2, 128),
    ((37, 29), (7, 5), (1, 1), (1, 1), (True, False), 2, 2, 32),          # token-permuted route (odd extents)
    ((10, 16, 24), (6, 8, 8), (1, 8, 4), (1, 1, 1), (True, False, False), 3, 3, 128),
    ((8, 16, 16), (8, 16, 16), (1, 1, 1), (1, 1, 1), (True, False, False), 1, 1, 64),
]


@pytest.mark.parametrize("case", QUEUE_CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_work_queue_launch_equals_one_workgroup_per_tile(case, dtype):
    # resident workgroups pulling Q tiles from per-XCD queues compute the same bits as a workgroup
    # per Q tile, on both operand layouts; twice in a row (the queues are cleared by every launch)
    shape, k, s, d, causal, H, Hkv, D = case
    q, kk, v = make_qkv(3, shape, H, Hkv, D, dtype, seed=11)
    with torch.no_grad():
        ref = amd_fna_generic(q, kk, v, k, s, d, causal, return_lse=True, run_persistent_kernel=False)  # anchored tiles
        for _ in range(2):
            got = amd_fna_generic(q, kk, v, k, s, d, causal, return_lse=True, run_persistent_kernel=True)
            assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
        perm = amd_fna_generic(q, kk, v, k, s, d, causal, return_lse=True, run_persistent_kernel=False, fused=False)
        got = amd_fna_generic(q, kk, v, k, s, d, causal, return_lse=True, run_persistent_kernel=True, fused=False)
        assert torch.equal(got[0], perm[0]) and torch.equal(got[1], perm[1])
    ref_o, ref_l = oracle_full(q, kk, v, k, s, d, causal)
    assert_close("out", to_np(got[0]), ref_o)
    assert_close("lse", to_np(got[1]), ref_l)
    # the wrapper zeroes its counter block once per (device, stream); every launch must leave it zeroed
    from natten_amd import _lib

    torch.cuda.synchronize()
    assert _lib._QUEUE_WORKSPACES and all(int(w.sum()) == 0 for w in _lib._QUEUE_WORKSPACES.values())


def test_work_queue_launch_many_more_tiles_than_workgroups():
    # 24 x 900 Q tiles against 512 resident workgroups, non-causal and causal, through the public API
    q, kk, v = make_qkv(1, (30, 48, 80), 4, 4, 128, torch.float16, seed=5)
    for causal in ((False, False, False), (True, False, False)):
        args = ((18, 24, 24), (16, 8, 8), (1, 1, 1), causal)
        with torch.no_grad():
            a = natten_amd.na3d(q, kk, v, *args, return_lse=True, run_persistent_kernel=True)
            b = natten_amd.na3d(q, kk, v, *args, return_lse=True, run_persistent_kernel=False)
            c = natten_amd.na3d(q, kk, v, *args, return_lse=True)  # the default picks one of the two
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
        assert torch.equal(c[0], b[0]) and torch.equal(c[1], b[1])


def test_work_queue_launch_replays_from_a_graph():
    # the launch clears its queues with a kernel, so the pair can be captured; replays with new
    # inputs and eager work in between give the eager bits every time
    q, kk, v = make_qkv(2, (32, 48), 2, 2, 64, torch.bfloat16, seed=9)
    args = ((9, 7), (2, 1), (1, 1), (False, False))
    sq, sk, sv = q.clone(), kk.clone(), v.clone()
    stream = torch.cuda.Stream()
    with torch.no_grad(), torch.cuda.stream(stream):
        amd_fna_generic(sq, sk, sv, *args, return_lse=True, run_persistent_kernel=True)  # warm up outside the capture
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            out, lse = amd_fna_generic(sq, sk, sv, *args, return_lse=True, run_persistent_kernel=True)
    for seed in (1, 2, 3):
        nq, nk, nv = make_qkv(2, (32, 48), 2, 2, 64, torch.bfloat16, seed=seed)
        sq.copy_(nq), sk.copy_(nk), sv.copy_(nv)
        g.replay()
        torch.cuda.synchronize()
        with torch.no_grad():
            eo, el = amd_fna_generic(nq, nk, nv, *args, return_lse=True, run_persistent_kernel=False)
        assert torch.equal(out, eo) and torch.equal(lse, el), f"replay {seed}"
