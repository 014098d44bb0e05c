"""GPU parity at the benchmark configurations' full sizes.

Where the oracle cannot evaluate every query in seconds, a seeded sample of query positions is
checked against the C oracle (all heads of each sampled query), and size-independent
properties cover the whole tensor: scaling V by a power of two scales the output bit-exactly
and leaves LSE unchanged; every output lies inside the range of V; token permute round trips
are bit-exact."""

import numpy as np
import pytest
import torch

import natten_amd
from oracle import c_oracle
from tests.gpu_utils import assert_close, make_qkv, oracle_full, to_np

pytestmark = pytest.mark.gpu


def _sampled_check(q, k, v, out, lse, kernel, stride, dilation, causal, n_samples, seed):
    B = q.shape[0]
    n = q.dim() - 3
    N = int(np.prod(q.shape[1 : 1 + n]))
    H, D = q.shape[-2], q.shape[-1]
    rng = np.random.default_rng(seed)
    tok = rng.integers(0, N, size=n_samples)
    # always include the corners, where windows are clamped
    tok[:2] = (0, N - 1)
    bat = rng.integers(0, B, size=n_samples)
    ref_o, ref_l, _ = c_oracle.na_rows(to_np(q), to_np(k), to_np(v), kernel, stride, dilation, causal, None, bat, tok,
                                       threads=8)
    ti, bi = torch.as_tensor(tok), torch.as_tensor(bat)
    got_o = to_np(out.reshape(B, N, H, D)[bi, ti])
    got_l = to_np(lse.reshape(B, N, H)[bi, ti])
    assert_close("sampled out", got_o, ref_o)
    assert_close("sampled lse", got_l, ref_l)


def _properties(fn, q, k, v, args, out, lse):
    with torch.no_grad():
        out2, lse2 = fn(q, k, v * 2, *args, return_lse=True)
    # exact for every normal number (a power-of-two factor commutes with each rounding); fp16
    # results below its normal range round differently before and after the doubling
    normal = out.float().abs() >= 2.0**-13 if out.dtype == torch.float16 else torch.ones_like(out, dtype=torch.bool)
    assert torch.equal(out2[normal], (out * 2)[normal]), "scaling V by two must scale the output bit-exactly"
    assert torch.allclose(out2.float(), out.float() * 2, atol=2.0**-13, rtol=0)
    assert torch.equal(lse2, lse), "LSE must not depend on V"
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    vmax = v.float().abs().max().item()
    assert out.float().abs().max().item() <= vmax * (1 + 1e-2)


@pytest.mark.parametrize("dil", [(1, 1), (2, 2)])
def test_config2_full(dil):
    q, k, v = make_qkv(2, (64, 64), 8, 8, 64, torch.bfloat16, seed=0)
    with torch.no_grad():
        out, lse = natten_amd.na2d(q, k, v, (13, 13), (1, 1), dil, return_lse=True)
    ref_o, ref_l = oracle_full(q, k, v, (13, 13), (1, 1), dil, (False, False))
    assert_close("out", to_np(out), ref_o)
    assert_close("lse", to_np(lse), ref_l)
    _properties(natten_amd.na2d, q, k, v, ((13, 13), (1, 1), dil), out, lse)


def test_config3_full_size_sampled():
    q, k, v = make_qkv(1, (128, 128), 16, 16, 128, torch.float16, seed=0, std=0.5)
    args = ((32, 32), (16, 16), (1, 1))
    with torch.no_grad():
        out, lse = natten_amd.na2d(q, k, v, *args, return_lse=True)
    _sampled_check(q, k, v, out, lse, *args, (False, False), n_samples=200, seed=1)
    _properties(natten_amd.na2d, q, k, v, args, out, lse)


def test_config4_full_size_sampled():
    q, k, v = make_qkv(1, (30, 48, 80), 24, 24, 128, torch.bfloat16, seed=0)
    args = ((18, 24, 24), (1, 8, 8), (1, 1, 1), (True, False, False))
    with torch.no_grad():
        out, lse = natten_amd.na3d(q, k, v, *args, return_lse=True)
    _sampled_check(q, k, v, out, lse, *args, n_samples=64, seed=2)
    _properties(natten_amd.na3d, q, k, v, args, out, lse)
    # causal in time: the first frame attends only itself, so its LSE is below the last frame's
    assert (lse[0, 0].mean() < lse[0, -1].mean()).item()


def test_permute_round_trip_full_size():
    q, _, _ = make_qkv(1, (30, 48, 80), 24, 24, 128, torch.bfloat16, seed=3)
    p, layout, post = natten_amd.token_permute_operation(q, (2, 8, 8), (1, 1, 1))
    assert post == (30, 48, 80)
    back = natten_amd.token_unpermute_operation(p, layout, (2, 8, 8), (1, 1, 1))
    assert torch.equal(back, q)
    # each tile of the permuted sequence is the (2, 8, 8) block it came from
    blk = q[0, 2:4, 8:16, 16:24]  # tile (1, 1, 2) -> index 1 + 15 * (1 + 6 * 2)
    idx = 1 + 15 * (1 + 6 * 2)
    tile = p[0, idx * 128 : (idx + 1) * 128].reshape(8, 8, 2, 24, 128)  # dimension 0 fastest
    assert torch.equal(tile.permute(2, 1, 0, 3, 4), blk)
