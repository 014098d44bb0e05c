"""GPU parity of the backward pass: gradients from the public API (autograd function over the
C ABI: delta, token permutes, dQ and dK/dV kernels) against the CPU oracle's float64 gradients on
the same (already rounded) inputs, with q, k, v, dO ~ N(0, 1).

Tolerance: fp16 atol = rtol = 1e-2; bf16 atol = rtol = 2e-2.  The kernels round P and
dS = P (dP - delta) to the operand type before the second matrix product, as the reference's
kernels do; |dP| ~ sqrt(head_dim), so one bf16 rounding of dS (2^-9 relative) is worth up to
~1e-2 in a gradient whose window holds few keys.  The reference's own bar is atol 1e-2, rtol 0
on gradients twenty times smaller (dO ~ 0.05 N(0, 1): tests/test_blackwell_fna.py:104-109,
tests/utils.py:117-120), i.e. ten times looser than this one."""

import numpy as np
import pytest
import torch

import natten_amd
from natten_amd.tile_config import get_all_backward_tile_shapes
from oracle import c_oracle
from oracle import na_oracle as O
from tests.gpu_utils import assert_close, make_qkv, routes_agree_bit_for_bit, to_np, tuplify

pytestmark = pytest.mark.gpu

NA = {1: natten_amd.na1d, 2: natten_amd.na2d, 3: natten_amd.na3d}
TOL = {torch.float16: 1e-2, torch.bfloat16: 2e-2}


def run_backward(B, H, Hkv, D, shape, k, s, d, causal, dtype, bq=None, bkv=None, seed=0):
    n = len(shape)
    k, s, d, causal = (tuplify(x, n) for x in (k, s, d, causal))
    q, kk, v = make_qkv(B, shape, H, Hkv, D, dtype, seed=seed)
    gen = torch.Generator().manual_seed(seed + 1000)
    d_out = torch.randn(q.shape, generator=gen).to(dtype).cuda()
    q.requires_grad_(True)
    kk.requires_grad_(True)
    v.requires_grad_(True)
    out = NA[n](q, kk, v, k, s, d, causal, backward_q_tile_shape=bq, backward_kv_tile_shape=bkv)
    out.backward(d_out)
    torch.cuda.synchronize()
    ref = c_oracle.na_backward(to_np(q), to_np(kk), to_np(v), to_np(d_out), k, s, d, causal)
    tag = f"{shape} k={k} s={s} d={d} c={causal} H={H}/{Hkv} D={D} {dtype} tiles={bq},{bkv}"
    for name, got, r in zip(("dq", "dk", "dv"), (q.grad, kk.grad, v.grad), ref):
        assert got is not None and got.dtype == dtype and got.shape == r.shape, name
        assert_close(f"{name} {tag}", to_np(got), r, atol=TOL[dtype], rtol=TOL[dtype])
    if not all(kk_ == x for kk_, x in zip(k, shape)) or any(causal):
        # whichever layout the backward above worked on (the original tensors when no extent needs
        # padding, token-permuted copies otherwise), the permuted route must agree bit for bit
        from natten_amd.fna import amd_fna_generic

        from natten_amd.tile_config import check_fna_forward_config

        grads = []
        for route in (dict(anchored_tiles=False), dict(fused=False)):
            q2, k2, v2 = (t.detach().clone().requires_grad_(True) for t in (q, kk, v))
            amd_fna_generic(q2, k2, v2, k, s, d, causal, backward_q_tile_shape=bq, backward_kv_tile_shape=bkv,
                            **route).backward(d_out)
            grads.append((q2.grad, k2.grad, v2.grad))
        # (the forward results the backward starts from are only bit-equal between the routes where
        # both place the keys alike in their tiles; elsewhere they agree up to summation order)
        _, fwd_kt = check_fna_forward_config(q, k, s, d, causal, None, None)
        exact = routes_agree_bit_for_bit(shape, d, fwd_kt)
        # ... and the backward on the original tensors sums in the permuted route's order only where its
        # own tiles divide the extents (elsewhere it moves the last tile of a dimension back)
        from natten_amd.tile_config import check_fna_backward_config
        bwd_tiles = check_fna_backward_config(q, k, s, d, causal, bq, bkv)
        exact = exact and all(X % (dd * t) == 0 for tile in bwd_tiles for X, dd, t in zip(shape, d, tile))
        for name, a, b, c in zip(("dq", "dk", "dv"), grads[0], grads[1], (q.grad, kk.grad, v.grad)):
            if exact:
                assert torch.equal(a, b), f"original-layout and permuted backward differ in {name}: {tag}"
            else:
                assert_close(f"routes {name} {tag}", to_np(a), to_np(b), atol=TOL[dtype], rtol=TOL[dtype])
            # and the default (KV tiles of the forward laid out from the window's first key): two
            # roundings of the same gradient, a unit of the last place apart at most
            assert_close(f"default route {name} {tag}", to_np(c), to_np(b), atol=1.5 * TOL[dtype], rtol=TOL[dtype])


@pytest.mark.parametrize("case", [
    # extents no tile shape divides, uneven dilation groups: the backward still runs on the original tensors
    (1, 2, 2, 64, (57, 20, 88), (5, 7, 9), (1, 2, 3), (2, 1, 1), (False, False, False)),
    (1, 4, 2, 128, (84, 69), (11, 9), (2, 1), (1, 1), (True, False)),
    (2, 2, 1, 32, (301,), (33,), (4,), (2,), (False,)),
    (1, 2, 2, 128, (11, 19, 37), (4, 6, 9), (1, 2, 4), (1, 1, 1), (True, False, True)),
])
def test_backward_odd_extents_on_the_original_tensors(case):
    from natten_amd import _lib
    from natten_amd.tile_config import check_fna_backward_config

    B, H, Hkv, D, shape, k, s, d, causal = case
    probe = torch.empty((B, *shape, H, D), dtype=torch.bfloat16, device="meta")
    bq, bkv = check_fna_backward_config(probe, k, s, d, causal, None, None)
    assert any(X % (dd * t) for tile in (bq, bkv) for X, dd, t in zip(shape, d, tile)), "the case is meant to need edge tiles"
    assert _lib.backward_fused_layout_supported(shape, d, bq, bkv, row_bytes=H * D * 2)
    run_backward(B, H, Hkv, D, shape, k, s, d, causal, torch.bfloat16, seed=31)
    run_backward(B, H, Hkv, D, shape, k, s, d, causal, torch.float16, seed=32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_backward_1d(dtype):
    run_backward(1, 2, 2, 32, (256,), 7, 1, 1, False, dtype)
    run_backward(2, 4, 2, 64, (300,), 33, 4, 2, True, dtype, seed=1)
    run_backward(1, 2, 1, 128, (77,), 9, 3, 1, False, dtype, seed=2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_backward_2d(dtype):
    run_backward(2, 2, 2, 64, (20, 24), (5, 7), (2, 1), (1, 2), (False, True), dtype, seed=3)
    run_backward(1, 4, 1, 128, (32, 32), (13, 13), (1, 1), (1, 1), (False, False), dtype, seed=4)
    run_backward(1, 2, 2, 48, (17, 19), (4, 6), (2, 3), (2, 1), (True, True), dtype, seed=5)  # head_dim padded to 64


def test_backward_3d():
    run_backward(1, 2, 1, 64, (9, 16, 24), (4, 8, 8), (1, 8, 4), 1, (True, False, False), torch.bfloat16, seed=6)
    # extents that are multiples of dilation x tile: the backward works on the original tensors
    run_backward(2, 4, 2, 128, (8, 16, 16), (3, 8, 8), (1, 4, 8), (2, 1, 1), (True, False, False), torch.bfloat16,
                 (2, 8, 8), (4, 4, 8), seed=60)
    run_backward(1, 2, 2, 64, (4, 32, 16), (2, 9, 5), (1, 3, 1), (1, 2, 1), (False, False, True), torch.float16,
                 (2, 16, 4), (1, 8, 16), seed=61)
    run_backward(1, 2, 2, 32, (6, 10, 9), (3, 4, 5), (1, 2, 2), (2, 1, 1), (False, True, False), torch.float16, seed=7)
    run_backward(2, 1, 1, 128, (8, 8, 8), (3, 3, 3), 1, 1, False, torch.bfloat16, seed=8)


def test_backward_every_tile_shape_2d():
    for i, (bq, bkv) in enumerate(get_all_backward_tile_shapes(2)):
        if i % 3 == 0:  # a third of the 64 pairs: every Q shape and every KV shape occurs
            run_backward(1, 2, 1, 32, (40, 36), (9, 6), (2, 1), (1, 2), (True, False), torch.bfloat16, bq, bkv, seed=i)


def test_backward_tile_shapes_3d():
    for bq, bkv in [((2, 8, 8), (2, 8, 8)), ((1, 8, 16), (4, 4, 8)), ((8, 4, 4), (1, 2, 64)), ((128, 1, 1), (1, 128, 1))]:
        run_backward(1, 2, 2, 64, (10, 12, 20), (4, 5, 6), (1, 2, 3), 1, (True, False, False), torch.float16, bq, bkv, seed=9)


def test_backward_random_sweep():
    rng = np.random.default_rng(77)
    done = 0
    while done < 16:
        n = int(rng.integers(1, 4))
        shape = tuple(int(rng.integers(4, {1: 300, 2: 36, 3: 12}[n])) for _ in range(n))
        d = tuple(int(rng.integers(1, max(2, x // 4 + 1))) for x in shape)
        if any(x // dd < 2 for x, dd in zip(shape, d)):
            continue
        k = tuple(int(rng.integers(2, x // dd + 1)) for x, dd in zip(shape, d))
        if all(kk * dd == x for kk, dd, x in zip(k, d, shape)) and n > 1:
            continue
        s = tuple(int(rng.integers(1, kk + 1)) for kk in k)
        causal = tuple(bool(rng.integers(0, 2)) for _ in range(n))
        Hkv = int(rng.choice([1, 2]))
        H = Hkv * int(rng.choice([1, 2]))
        D = int(rng.choice([32, 64, 128]))
        run_backward(1, H, Hkv, D, shape, k, s, d, causal, [torch.bfloat16, torch.float16][done % 2], seed=done)
        done += 1


@pytest.mark.parametrize("case", [
    # (H, Hkv, D, shape, k, s, d, causal, seed): windows of one or two keys, where a probability is 1
    # or close to it.  Formed from other logits than the forward's (queries scaled after the matrix
    # product instead of before it), such a probability came out as 1 +- 0.5 % and dv missed the
    # tolerance by up to a factor of two; formed from the forward's own operand it is exact.
    (4, 2, 64, (24,), (3,), (1,), (3,), (True,), 27693),
    (2, 1, 64, (55,), (2,), (2,), (13,), (True,), 27895),
    (2, 1, 128, (230,), (10,), (5,), (16,), (True,), 27897),
    (4, 2, 64, (34, 28), (2, 3), (2, 2), (7, 5), (True, True), 28641),
    (2, 1, 32, (7, 10, 10), (2, 10, 2), (2, 1, 2), (1, 1, 1), (True, True, True), 27707),
])
def test_backward_uses_the_forward_logits(case):
    H, Hkv, D, shape, k, s, d, causal, seed = case
    run_backward(1, H, Hkv, D, shape, k, s, d, causal, torch.bfloat16, seed=seed)


ATTN_CASES = [
    # B, Sq, Skv, H, Hkv, D, causal
    (2, 128, 128, 2, 2, 64, False),
    (1, 125, 300, 2, 1, 128, False),
    (1, 300, 125, 4, 2, 32, True),   # top-left causal, more queries than keys
    (1, 77, 77, 3, 3, 64, True),
    (1, 5, 1, 2, 2, 64, False),
    (1, 130, 9, 4, 2, 48, False),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_attention_backward(dtype):
    for i, (B, Sq, Skv, H, Hkv, D, causal) in enumerate(ATTN_CASES):
        gen = torch.Generator().manual_seed(i)
        q = torch.randn((B, Sq, H, D), generator=gen).to(dtype).cuda().requires_grad_(True)
        k = torch.randn((B, Skv, Hkv, D), generator=gen).to(dtype).cuda().requires_grad_(True)
        v = torch.randn((B, Skv, Hkv, D), generator=gen).to(dtype).cuda().requires_grad_(True)
        d_out = torch.randn((B, Sq, H, D), generator=gen).to(dtype).cuda()
        out, lse = natten_amd.attention(q, k, v, is_causal=causal, return_lse=True)
        out.backward(d_out)
        ref = O.attention_backward(to_np(q), to_np(k), to_np(v), to_np(d_out), is_causal=causal)
        tag = f"attention {(B, Sq, Skv, H, Hkv, D, causal)} {dtype}"
        for name, got, r in zip(("dq", "dk", "dv"), (q.grad, k.grad, v.grad), ref):
            assert_close(f"{name} {tag}", to_np(got), r, atol=TOL[dtype], rtol=TOL[dtype])


def test_full_window_backward_takes_the_attention_path():
    q, kk, v = make_qkv(1, (8, 12), 2, 2, 64, torch.float16, seed=3)
    d_out = torch.randn(q.shape, generator=torch.Generator().manual_seed(5)).to(q.dtype).cuda()
    for t in (q, kk, v):
        t.requires_grad_(True)
    natten_amd.na2d(q, kk, v, (8, 12)).backward(d_out)
    ref = O.na_backward(to_np(q), to_np(kk), to_np(v), to_np(d_out), (8, 12))
    for name, got, r in zip(("dq", "dk", "dv"), (q.grad, kk.grad, v.grad), ref):
        assert_close(name, to_np(got), r)


def test_compute_delta_matches_numpy():
    from natten_amd import _lib

    for D in (32, 64, 128):
        gen = torch.Generator().manual_seed(D)
        o = torch.randn((3, 37, 5, D), generator=gen).to(torch.bfloat16).cuda()
        do = torch.randn((3, 37, 5, D), generator=gen).to(torch.bfloat16).cuda()
        got = _lib.compute_delta(o, do)
        ref = (to_np(o).astype(np.float64) * to_np(do)).sum(-1)
        assert got.dtype == torch.float32 and got.shape == o.shape[:-1]
        assert_close(f"delta D={D}", to_np(got), ref, atol=1e-4, rtol=1e-5)


def test_backward_is_deterministic():
    q, kk, v = make_qkv(1, (24, 24), 2, 1, 64, torch.bfloat16, seed=11)
    d_out = torch.randn(q.shape, generator=torch.Generator().manual_seed(12)).to(q.dtype).cuda()
    grads = []
    for _ in range(2):
        qq, k2, v2 = (t.clone().requires_grad_(True) for t in (q, kk, v))
        natten_amd.na2d(qq, k2, v2, (7, 5), (2, 1), is_causal=(True, False)).backward(d_out)
        grads.append((qq.grad, k2.grad, v2.grad))
    for a, b in zip(*grads):
        assert torch.equal(a, b)


def test_backward_argument_errors():
    q, kk, v = make_qkv(1, (16, 16), 2, 2, 32, torch.bfloat16, seed=0)
    q.requires_grad_(True)
    with pytest.raises(ValueError):
        natten_amd.na2d(q, kk, v, 3, backward_q_tile_shape=(8, 8), backward_kv_tile_shape=(8, 16))
    with pytest.raises(ValueError):
        natten_amd.na2d(q, kk, v, 3, backward_q_tile_shape=(8, 16))
    q8 = torch.zeros(1, 16, 16, 2, 32).to(torch.float8_e4m3fn).cuda().requires_grad_(True)
    with pytest.raises(NotImplementedError):  # no backward for 8-bit operands
        natten_amd.na2d(q8, q8, q8, 3)


@pytest.mark.parametrize("out_dtype", [None, torch.float32])
@pytest.mark.parametrize("na_dim,D", [(1, 64), (2, 48), (3, 128)])
def test_backward_with_additional_keys_values(na_dim, D, out_dtype):
    # the merge hands both partial attentions the merged output and LSE, so that their backward
    # passes add up to the backward of attention over the joint context (reference
    # src/natten/attn_merge.py:130-190); checked against the dense oracle on the concatenated keys
    shape = {1: (100,), 2: (12, 20), 3: (5, 8, 12)}[na_dim]
    ks = {1: (9,), 2: (5, 7), 3: (3, 3, 5)}[na_dim]
    causal = {1: (True,), 2: (False, True), 3: (False, False, False)}[na_dim]
    dtype = torch.float16
    q, kk, v = make_qkv(2, shape, 4, 2, D, dtype, seed=17)
    gen = torch.Generator().manual_seed(18)
    ak = torch.randn((2, 37, 2, D), generator=gen).to(dtype).cuda()
    av = torch.randn((2, 37, 2, D), generator=gen).to(dtype).cuda()
    d_out = torch.randn(q.shape, generator=gen).to(dtype).cuda()
    for t in (q, kk, v, ak, av):
        t.requires_grad_(True)
    # with an output type other than the operands' the partial results must still reach the merge
    # uncast (the merge's backward writes into the tensors the partial attentions saved)
    out = NA[na_dim](q, kk, v, ks, is_causal=causal, additional_keys=ak, additional_values=av, out_dtype=out_dtype)
    assert out.dtype == (out_dtype or dtype)
    out.backward(d_out.to(out.dtype))
    N = int(np.prod(shape))
    B, H = q.shape[0], q.shape[-2]
    mask = np.concatenate([O.na_mask_dense(shape, ks, 1, 1, causal), np.ones((N, 37), dtype=bool)], axis=1)
    k_all = np.concatenate([to_np(kk).reshape(B, N, 2, D), to_np(ak)], axis=1)
    v_all = np.concatenate([to_np(v).reshape(B, N, 2, D), to_np(av)], axis=1)
    dq, dk, dv = O.masked_attention_backward(to_np(q).reshape(B, N, H, D), k_all, v_all, to_np(d_out).reshape(B, N, H, D),
                                             mask, float(D) ** -0.5)
    refs = {"dq": dq.reshape(q.shape), "dk": dk[:, :N].reshape(kk.shape), "dv": dv[:, :N].reshape(v.shape),
            "dak": dk[:, N:], "dav": dv[:, N:]}
    got = {"dq": q.grad, "dk": kk.grad, "dv": v.grad, "dak": ak.grad, "dav": av.grad}
    for name in refs:
        assert_close(f"{name} na{na_dim}d D={D}", to_np(got[name]), refs[name], atol=TOL[dtype], rtol=TOL[dtype])


def test_layer_trains():
    # the layer's parameters and input receive finite gradients of the right shape, and they
    # agree with the same computation assembled from linear layers and the oracle's attention gradient
    torch.manual_seed(0)
    layer = natten_amd.NeighborhoodAttention2D(embed_dim=64, num_heads=2, kernel_size=(5, 3), stride=(1, 1),
                                               is_causal=(False, True)).cuda().to(torch.bfloat16)
    x = torch.randn(2, 12, 10, 64, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    y = layer(x)
    y.float().square().mean().backward()
    assert x.grad is not None and x.grad.shape == x.shape and torch.isfinite(x.grad).all()
    for name, prm in layer.named_parameters():
        assert prm.grad is not None and torch.isfinite(prm.grad).all(), name
        assert prm.grad.abs().max() > 0, name


def _pairs(B, H, shape, k):
    n = 1
    for x in shape:
        n *= x
    w = 1
    for x in k:
        w *= x
    return B * H * n * w


@pytest.mark.parametrize("na_dim", [1, 2, 3])
def test_reference_problem_lists_backward(na_dim):
    # the hand-picked problems of the reference's test-suite (tests/problems.py), forward + backward
    # as tests/test_blackwell_fna.py runs them, each non-causal and causal along its first
    # dimension; the largest ones (more than 6e7 query-key pairs for the float64 oracle) run in
    # test_large_reference_problems_backward_sampled below
    from tests import problems

    cases = {1: problems.NA_1D, 2: problems.NA_2D, 3: problems.NA_3D}[na_dim]
    ran = 0
    for i, (B, H, Hkv, D, shape, k, s, d) in enumerate(cases):
        if _pairs(B, H, shape, k) > 6e7:
            continue
        dtype = torch.bfloat16 if i % 2 == 0 else torch.float16
        for causal in ((False,) * na_dim, (True,) + (False,) * (na_dim - 1)):
            run_backward(B, H, Hkv, D, shape, k, s, d, causal, dtype, seed=100 + i)
            ran += 1
    assert ran >= 16


def _large_backward_cases():
    from tests import problems

    cases = []
    for na_dim, lst in ((1, problems.NA_1D), (2, problems.NA_2D), (3, problems.NA_3D)):
        cases += [(na_dim, i, c) for i, c in enumerate(lst) if _pairs(c[0], c[1], c[4], c[5]) > 6e7]
    # the long 1-D problems of the reference's profiler tests (tests/problems.py NA_1D_LONG): both ends of the strides
    cases += [(1, 100 + i, c) for i, c in enumerate(problems.NA_1D_LONG) if c[6] in ((2048,), (1,))]
    return cases


@pytest.mark.parametrize("na_dim,idx,case", _large_backward_cases())
def test_large_reference_problems_backward_sampled(na_dim, idx, case):
    # the reference problems too large for the whole-tensor float64 oracle: gradients at a stratified
    # sample of positions (corners, borders, stride-group and causal boundaries, random ones) against
    # the backward formulas in float64, non-causal and causal along the first dimension
    from tests.gpu_utils import sampled_backward_check

    B, H, Hkv, D, shape, k, s, d = case
    dtype = torch.bfloat16 if idx % 2 == 0 else torch.float16
    for causal in ((False,) * na_dim, (True,) + (False,) * (na_dim - 1)):
        q, kk, v = make_qkv(B, shape, H, Hkv, D, dtype, seed=300 + idx)
        gen = torch.Generator().manual_seed(1300 + idx)
        d_out = torch.randn(q.shape, generator=gen).to(dtype).cuda()
        for t in (q, kk, v):
            t.requires_grad_(True)
        out, lse = NA[na_dim](q, kk, v, k, s, d, causal, return_lse=True)
        out.backward(d_out)
        torch.cuda.synchronize()
        tag = f"{shape} k={k} s={s} d={d} c={causal} H={H}/{Hkv} D={D} {dtype}"
        sampled_backward_check(q.detach(), kk.detach(), v.detach(), d_out, out.detach(), lse.detach(), q.grad, kk.grad,
                               v.grad, k, s, d, causal, n_samples=48, seed=idx, atol=TOL[dtype], rtol=TOL[dtype],
                               tag=tag)


def test_backward_tile_shapes_per_launch_match_oracle_and_common_tiles():
    # on the original tensors the dq launch and the dk / dv launch take tile shapes of their own by
    # default; the gradients meet the oracle like those of any other tile shapes, and each launch
    # alone (C ABI `roles`) writes only its own results
    from natten_amd import _lib
    from natten_amd.tile_config import choose_backward_role_tile_shapes

    B, H, Hkv, D, shape, k, s, d, causal = 1, 4, 2, 128, (12, 16, 32), (7, 8, 8), (1, 8, 8), (1, 1, 1), (True, False, False)
    roles = choose_backward_role_tile_shapes(shape, k, s, d, causal)
    assert roles is not None and roles[0] != roles[1]
    run_backward(B, H, Hkv, D, shape, k, s, d, causal, torch.bfloat16, seed=21)   # default: per-launch shapes
    run_backward(B, H, Hkv, D, shape, k, s, d, causal, torch.float16, bq=roles[0][0], bkv=roles[0][1], seed=22)
    # the two launches one at a time
    q, kk, v = make_qkv(B, shape, H, Hkv, D, torch.bfloat16, seed=23)
    gen = torch.Generator().manual_seed(24)
    d_out = torch.randn(q.shape, generator=gen).to(torch.bfloat16).cuda()
    with torch.no_grad():
        out, lse = NA[3](q, kk, v, k, s, d, causal, return_lse=True)
        delta = _lib.compute_delta(out, d_out)
        both = _lib.fna_backward_fused(q, kk, v, d_out, lse, delta, k, s, d, causal, D ** -0.5, *roles[0], *roles[1])
        only_dq = _lib.fna_backward_fused(q, kk, v, d_out, lse, delta, k, s, d, causal, D ** -0.5, *roles[0])
        only_kv = _lib.fna_backward_fused(q, kk, v, d_out, lse, delta, k, s, d, causal, D ** -0.5, *roles[1])
    assert torch.equal(both[0], only_dq[0])                                   # dq: the dq launch's shapes
    assert torch.equal(both[1], only_kv[1]) and torch.equal(both[2], only_kv[2])  # dk, dv: the other launch's
