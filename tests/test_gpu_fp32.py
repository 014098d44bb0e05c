"""Float32 operands through the public ops (GPU): the forward kernel of its own for this type
against the float64 oracle at the tolerance the reference's tests state for float32
(tests/test_fna.py:107-131: atol 1e-4 on the output; the LSE is held to the same bar)."""

import numpy as np
import pytest
import torch

from natten_amd.functional import na1d, na2d, na3d
from tests.gpu_utils import assert_close, oracle_full, sampled_check, to_np

pytestmark = pytest.mark.gpu

NA = {1: na1d, 2: na2d, 3: na3d}
ATOL32 = 1e-4


def make(B, shape, H, Hkv, D, seed):
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn((B, *shape, H, D), generator=gen)
    k = torch.randn((B, *shape, Hkv, D), generator=gen)
    v = torch.randn((B, *shape, Hkv, D), generator=gen)
    return q.cuda(), k.cuda(), v.cuda()


def test_config1_na1d_fp32():
    # the configuration the reference runs on the CPU: B=1, heads=2, L=256, head_dim=32, kernel_size=7, seed 0
    q, k, v = make(1, (256,), 2, 2, 32, seed=0)
    out, lse = na1d(q, k, v, 7, return_lse=True)
    assert out.dtype == torch.float32 and out.shape == q.shape and lse.shape == q.shape[:-1]
    ref_o, ref_l = oracle_full(q, k, v, (7,), (1,), (1,), (False,))
    assert_close("out", to_np(out), ref_o, atol=ATOL32, rtol=ATOL32)
    assert_close("lse", to_np(lse), ref_l, atol=ATOL32, rtol=ATOL32)


CASES = [
    # B, shape, H, Hkv, D, kernel, stride, dilation, causal
    (2, (300,), 4, 2, 32, (33,), (4,), (2,), (True,)),
    (1, (1000,), 2, 2, 64, (128,), (16,), (3,), (False,)),
    (1, (19, 23), 3, 1, 64, (5, 8), (2, 3), (2, 1), (False, True)),
    (2, (16, 32), 2, 2, 128, (16, 9), (1, 4), (1, 2), (True, False)),
    (1, (6, 10, 12), 2, 2, 32, (3, 5, 4), (1, 2, 2), (2, 1, 1), (True, False, False)),
    (1, (8, 8, 16), 2, 1, 16, (8, 8, 16), (1, 1, 1), (1, 1, 1), (False, False, False)),   # window = whole input
    (1, (9, 7, 11), 1, 1, 40, (4, 3, 5), (2, 1, 3), (1, 2, 1), (False, False, True)),     # padded head dim
]


@pytest.mark.parametrize("case", CASES)
def test_fp32_problems_match_oracle(case):
    B, shape, H, Hkv, D, kernel, stride, dilation, causal = case
    q, k, v = make(B, shape, H, Hkv, D, seed=len(shape) * 7 + D)
    out, lse = NA[len(shape)](q, k, v, kernel, stride=stride, dilation=dilation, is_causal=causal, return_lse=True)
    assert out.dtype == torch.float32
    ref_o, ref_l = oracle_full(q, k, v, kernel, stride, dilation, causal)
    tag = f"{shape} k={kernel} s={stride} d={dilation} c={causal} H={H}/{Hkv} D={D}"
    assert_close("out " + tag, to_np(out), ref_o, atol=ATOL32, rtol=ATOL32)
    assert_close("lse " + tag, to_np(lse), ref_l, atol=ATOL32, rtol=ATOL32)


def test_fp32_large_sampled_and_scale_properties():
    # a problem of c2's shape at float32, by stratified samples; doubling V doubles O bit-exactly
    q, k, v = make(2, (64, 64), 8, 8, 64, seed=3)
    out, lse = na2d(q, k, v, (13, 13), return_lse=True)
    sampled_check(q, k, v, out, lse, (13, 13), (1, 1), (1, 1), (False, False), 600, seed=4, atol=ATOL32, rtol=ATOL32)
    out2, lse2 = na2d(q, k, 2 * v, (13, 13), return_lse=True)
    assert torch.equal(out2, 2 * out) and torch.equal(lse2, lse)


def test_fp32_explicit_scale_and_tiles():
    q, k, v = make(1, (32, 32), 2, 2, 32, seed=5)
    out, lse = na2d(q, k, v, (7, 7), scale=0.37, q_tile_shape=(4, 32), kv_tile_shape=(2, 32), return_lse=True)
    ref_o, ref_l = oracle_full(q, k, v, (7, 7), (1, 1), (1, 1), (False, False), 0.37)
    assert_close("out", to_np(out), ref_o, atol=ATOL32, rtol=ATOL32)
    assert_close("lse", to_np(lse), ref_l, atol=ATOL32, rtol=ATOL32)


def test_fp32_limits_are_reported():
    q, k, v = make(1, (64,), 2, 2, 32, seed=6)
    with pytest.raises((ValueError, RuntimeError)):      # only tiles of 128 x 64 tokens
        na1d(q, k, v, 7, q_tile_shape=(256,), kv_tile_shape=(64,))
    qg = q.clone().requires_grad_(True)
    with pytest.raises(NotImplementedError):             # forward only
        na1d(qg, k, v, 7)
    with pytest.raises((NotImplementedError, ValueError)):  # no dequantisation scales for float32
        na1d(q, k, v, 7, q_scale=2.0)
    extra = torch.randn((1, 16, 2, 32), device="cuda")
    with pytest.raises(NotImplementedError):             # dense attention (the additional keys' path) has no float32 form
        na1d(q, k, v, 7, additional_keys=extra, additional_values=extra)
