"""KV-split launches of the forward kernel (GPU): several workgroups share the KV tiles of a Q tile
and their partial results are merged.  Checked against the float64 oracle at the bar of the
unsplit kernel, against the unsplit launch, with runs that hold none of a query's keys (causal
windows, more splits than tiles), and through the default the public ops pick for small grids."""

import pytest
import torch

from natten_amd import _lib
from natten_amd.fna import amd_fna_generic
from natten_amd.functional import kv_splits_default, na1d, na2d, na3d
from natten_amd.tile_config import check_fna_forward_config
from tests.gpu_utils import assert_close, make_qkv, oracle_full, sampled_check, to_np

pytestmark = pytest.mark.gpu

NA = {1: na1d, 2: na2d, 3: na3d}

CASES = [
    # B, shape, H, Hkv, D, kernel, stride, dilation, causal, dtype, splits
    (1, (1024,), 2, 2, 128, (512,), (1,), (1,), (False,), torch.float16, 2),
    (1, (1024,), 2, 1, 64, (512,), (64,), (1,), (True,), torch.bfloat16, 8),     # first Q tiles: fewer tiles than splits
    (1, (1500,), 1, 1, 32, (300,), (7,), (2,), (False,), torch.bfloat16, 3),     # ragged extent, dilation
    (2, (24, 40), 2, 2, 128, (17, 24), (1, 8), (1, 1), (False, False), torch.float16, 4),
    (1, (20, 36), 2, 2, 64, (9, 20), (2, 3), (1, 1), (True, False), torch.bfloat16, 2),
    (1, (6, 12, 16), 2, 1, 128, (5, 12, 9), (1, 4, 1), (1, 1, 1), (False, False, True), torch.bfloat16, 5),
]


@pytest.mark.parametrize("case", CASES)
def test_split_launch_matches_oracle_and_unsplit_launch(case):
    B, shape, H, Hkv, D, kernel, stride, dilation, causal, dtype, splits = case
    q, k, v = make_qkv(B, shape, H, Hkv, D, dtype, seed=len(shape) + splits)
    tag = f"{shape} k={kernel} s={stride} d={dilation} c={causal} D={D} splits={splits}"
    print(tag, flush=True)
    whole_o, whole_l = amd_fna_generic(q, k, v, kernel, stride, dilation, causal, return_lse=True, kv_splits=1)
    out, lse = amd_fna_generic(q, k, v, kernel, stride, dilation, causal, return_lse=True, kv_splits=splits)
    assert out.shape == q.shape and out.dtype == dtype and lse.shape == q.shape[:-1]
    ref_o, ref_l = oracle_full(q, k, v, kernel, stride, dilation, causal)
    assert_close("out " + tag, to_np(out), ref_o)
    assert_close("lse " + tag, to_np(lse), ref_l)
    # against the one-workgroup-per-tile result: the partial outputs are rounded to the operand type
    # before the merge (2^-8 relative for bf16, 2^-11 for fp16), nothing else differs
    eps = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    assert_close("out vs unsplit " + tag, to_np(out), to_np(whole_o), atol=eps, rtol=eps)
    assert_close("lse vs unsplit " + tag, to_np(lse), to_np(whole_l), atol=1e-5, rtol=1e-5)


def test_partial_results_of_the_split_entry_point():
    # through the C ABI: parts are normalised over their own keys; a run with none of a query's keys
    # holds zeros and -inf; the merge of all parts is the whole attention
    shape, kernel, causal = (1024,), (256,), (True,)
    q, k, v = make_qkv(1, shape, 2, 2, 64, torch.float16, seed=5)
    qt, kt = check_fna_forward_config(q, kernel, (1,), (1,), causal, None, None)
    parts, lses = _lib.fna_forward_fused_split(q, k, v, kernel, (1,), (1,), causal, 64 ** -0.5, qt, kt, 4)
    assert parts.shape == (4, *q.shape) and lses.shape == (4, *q.shape[:-1])
    # the first query attends only key 0: one KV tile, so three of the four runs are empty for it
    first = lses[:, 0, 0, :]
    assert int(torch.isinf(first).sum()) == 3 * first.shape[-1] and bool(torch.isfinite(first).any(dim=0).all())
    assert bool((parts[:, 0, 0][torch.isinf(first)] == 0).all())
    assert bool(torch.isfinite(parts.float()).all()) and not bool(torch.isnan(lses).any())
    out, lse = _lib.merge_parts(parts, lses)
    # the same by two-way merges (more roundings of the intermediate outputs, same LSE)
    o2, l2 = parts[0], lses[0]
    for i in range(1, 4):
        o2, l2 = _lib.merge_two(o2, l2, parts[i], lses[i])
    assert_close("merge_parts vs merge_two, out", to_np(out), to_np(o2), atol=2.0 ** -9, rtol=2.0 ** -9)
    assert_close("merge_parts vs merge_two, lse", to_np(lse), to_np(l2), atol=1e-5, rtol=1e-5)
    ref_o, ref_l = oracle_full(q, k, v, kernel, (1,), (1,), causal)
    assert_close("out", to_np(out), ref_o)
    assert_close("lse", to_np(lse), ref_l)
    # total probability mass: exp(lse) is the sum of the parts' exp(lse)
    assert_close("lse = logsumexp of the parts", to_np(torch.logsumexp(lses, dim=0)), to_np(lse), atol=1e-5, rtol=1e-5)


def test_default_splits_a_small_grid_with_long_windows():
    # one head, 64 Q tiles of 34 KV tiles each: the public op splits four ways by itself
    shape, kernel = (8192,), (2048,)
    q, k, v = make_qkv(1, shape, 1, 1, 128, torch.float16, seed=9)
    qt, kt = check_fna_forward_config(q, kernel, (1,), (1,), (False,), None, None)
    assert kv_splits_default(1, 1, shape, kernel, (1,), (1,), (False,), qt, kt) == 4
    assert kv_splits_default(1, 2, shape, kernel, (1,), (1,), (False,), qt, kt) == 2
    # (not with 256 Q tiles, not with short or causal windows)
    assert kv_splits_default(1, 1, (32768,), kernel, (1,), (1,), (False,), qt, kt) == 1
    assert kv_splits_default(1, 1, shape, (256,), (1,), (1,), (False,), qt, kt) == 1
    assert kv_splits_default(1, 1, shape, kernel, (1,), (1,), (True,), qt, kt) == 1
    out, lse = na1d(q, k, v, kernel, return_lse=True)
    sampled_check(q, k, v, out, lse, kernel, (1,), (1,), (False,), n_samples=300, seed=1)
    same_o, same_l = amd_fna_generic(q, k, v, kernel, 1, 1, False, return_lse=True, kv_splits=4)
    assert torch.equal(out, same_o) and torch.equal(lse, same_l)
    # gradients flow through the split forward (the backward takes the merged output and LSE)
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q[:, :2048], k[:, :2048], v[:, :2048]))
    o = na1d(qg, kg, vg, (1024,))
    o.float().square().sum().backward()
    assert all(bool(torch.isfinite(t.grad.float()).all()) for t in (qg, kg, vg))


def test_split_limits():
    q, k, v = make_qkv(1, (512,), 1, 1, 64, torch.float16, seed=2)
    with pytest.raises(ValueError, match="kv_splits"):
        amd_fna_generic(q, k, v, (128,), kv_splits=9)
    with pytest.raises(ValueError, match="kv_splits"):
        amd_fna_generic(q, k, v, (128,), kv_splits=2, fused=False)
    with pytest.raises(ValueError, match="kv_splits"):
        amd_fna_generic(q, k, v, (128,), kv_splits=2, q_tile_shape=(64,), kv_tile_shape=(64,))
    q8 = q.to(torch.float8_e4m3fn)
    with pytest.raises(ValueError, match="kv_splits"):
        amd_fna_generic(q8, q8, q8, (128,), kv_splits=2, q_scale=1.0, k_scale=1.0, v_scale=1.0)
    qt, kt = check_fna_forward_config(q, (128,), (1,), (1,), (False,), None, None)
    with pytest.raises(RuntimeError, match="kv_splits"):
        _lib.fna_forward_fused_split(q, k, v, (128,), (1,), (1,), (False,), 0.125, qt, kt, 1)


@pytest.mark.parametrize("n", [1, 2, 3])
def test_split_random_sweep(n):
    # 40 random legal problems per rank (drawn like the reference's sweep), 2 .. 8 splits: the merged
    # result against the oracle, and against the unsplit launch up to the rounding of the partial outputs
    import numpy as np

    from tests.test_gpu_fna import _random_problem

    rng = np.random.default_rng(77 + n)
    for case in range(40):
        B, H, Hkv, D, shape, k, s, d, causal = _random_problem(rng, n)
        if all(kk == x for kk, x in zip(k, shape)) and not any(causal):
            continue  # the dense-attention shortcut of the public ops, not this kernel
        dtype = [torch.bfloat16, torch.float16][case % 2]
        splits = int(rng.integers(2, 9))
        q, kk_, v = make_qkv(B, shape, H, Hkv, D, dtype, seed=case)
        tag = f"{shape} k={k} s={s} d={d} c={causal} H={H}/{Hkv} D={D} {dtype} splits={splits}"
        print(tag, flush=True)
        whole_o, whole_l = amd_fna_generic(q, kk_, v, k, s, d, causal, return_lse=True, kv_splits=1)
        out, lse = amd_fna_generic(q, kk_, v, k, s, d, causal, return_lse=True, kv_splits=splits)
        cost = B * H * int(np.prod(shape)) * int(np.prod(k))
        if cost < 3e7:
            ref_o, ref_l = oracle_full(q, kk_, v, k, s, d, causal)
            assert_close("out " + tag, to_np(out), ref_o)
            assert_close("lse " + tag, to_np(lse), ref_l)
        else:
            sampled_check(q, kk_, v, out, lse, k, s, d, causal, 300, seed=case + 500, tag=tag)
        eps = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
        assert_close("out vs unsplit " + tag, to_np(out), to_np(whole_o), atol=eps, rtol=eps)
        assert_close("lse vs unsplit " + tag, to_np(lse), to_np(whole_l), atol=1e-5, rtol=1e-5)
