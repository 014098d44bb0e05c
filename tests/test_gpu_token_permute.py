"""GPU parity: token permute / unpermute through the C ABI, bit-exact against the oracle."""

import numpy as np
import pytest
import torch

import natten_amd
from oracle import na_oracle as O
from tests import problems

pytestmark = pytest.mark.gpu


def _payload(shape, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    if dtype == torch.uint8:  # stands for any 1-byte payload (fp8)
        return torch.randint(0, 256, shape, generator=gen, dtype=torch.uint8)
    return torch.randn(shape, generator=gen).to(dtype)


@pytest.mark.parametrize("flip", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.uint8])
def test_permute_matches_oracle_bit_exact(flip, dtype):
    for i, (B, H, layout, Dh, tile, dil) in enumerate(problems.PERMUTE):
        B, H = 2, 3
        if int(np.prod(layout)) * Dh > 2_000_000:
            Dh = 8
        x = _payload((B, *layout, H, Dh), dtype, i)
        xd = x.cuda()
        y, tl, post = natten_amd.token_permute_operation(xd, tile, dil, flip_tiled_dims=flip)
        xn = x.view(torch.int16).numpy() if dtype in (torch.float16, torch.bfloat16) else x.numpy()
        ref, tl_ref, post_ref = O.token_permute(xn, tile, dil, flip)
        yn = y.cpu()
        yn = yn.view(torch.int16).numpy() if dtype in (torch.float16, torch.bfloat16) else yn.numpy()
        assert tl == tl_ref and post == post_ref
        assert yn.shape == ref.shape, (layout, tile, dil)
        assert np.array_equal(yn.view(np.uint8), ref.view(np.uint8)), (layout, tile, dil, flip, dtype)
        back = natten_amd.token_unpermute_operation(y, tl, tile, dil, flip_tiled_dims=flip)
        assert back.shape == x.shape
        assert torch.equal(back.cpu().view(torch.uint8), x.contiguous().view(torch.uint8)), (layout, tile, dil, flip)


def test_unpermute_lse_shaped_rows():
    # rows of H float32 values (the LSE path: [B*G, S', H, 1]) take the narrow-vector route
    x = torch.randn(2, 9, 10, 3, 1)
    y, tl, _ = natten_amd.token_permute_operation(x.cuda(), (2, 4), (2, 1))
    ref, _, _ = O.token_permute(x.numpy(), (2, 4), (2, 1), True)
    assert np.array_equal(y.cpu().numpy(), ref)
    back = natten_amd.token_unpermute_operation(y, tl, (2, 4), (2, 1))
    assert torch.equal(back.cpu(), x)


def test_permute_rejects_bad_arguments():
    x = torch.randn(1, 8, 8, 2, 8).cuda()
    with pytest.raises(ValueError):
        natten_amd.token_permute_operation(x, (4,), None)
    with pytest.raises(ValueError):
        natten_amd.token_permute_operation(x, (4, 4), (2,))
    with pytest.raises(ValueError):
        natten_amd.token_unpermute_operation(torch.randn(3, 16, 2, 8).cuda(), (8, 8), (4, 4), (2, 1))
