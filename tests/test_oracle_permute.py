"""Pins the oracle's token permute / unpermute index map (no GPU).

The index-formula implementation is compared with an independent pad/reshape/transpose
restatement, with a third restatement in torch views, and through round trips, on the
reference's own problem tuples (tests/test_token_permute.py, used as data).
"""

import numpy as np
import pytest
import torch

from oracle import na_oracle as O
from tests import problems


def _torch_views(x, tile, dil, flip):
    # pad -> view [B, (R, t, d) per dim, H, Dh] -> permute -> reshape, written with torch ops.
    n = x.dim() - 3
    layout = x.shape[1 : 1 + n]
    R = [-(-(-(-X // t)) // d) for X, t, d in zip(layout, tile, dil)]
    padded = [r * t * d for r, t, d in zip(R, tile, dil)]
    pads = [0, 0, 0, 0]
    for X, P in reversed(list(zip(layout, padded))):
        pads += [0, P - X]
    xp = torch.nn.functional.pad(x, pads)
    split = []
    for r, t, d in zip(R, tile, dil):
        split += [r, t, d]
    xv = xp.view(x.shape[0], *split, x.shape[-2], x.shape[-1])
    dims = list(range(n))[::-1] if flip else list(range(n))
    perm = [0] + [3 * a + 3 for a in dims] + [3 * a + 1 for a in dims] + [3 * a + 2 for a in dims]
    perm += [3 * n + 1, 3 * n + 2]
    G = int(np.prod(dil))
    return xv.permute(*perm).reshape(x.shape[0] * G, -1, x.shape[-2], x.shape[-1]).contiguous()


@pytest.mark.parametrize("flip", [True, False])
def test_permute_three_restatements_agree(flip):
    for i, (B, H, layout, Dh, tile, dil) in enumerate(problems.PERMUTE):
        if int(np.prod(layout)) * Dh > 4_000_000:
            Dh = 4
        dil = dil or tuple([1] * len(layout))
        rng = np.random.default_rng(i)
        x = rng.standard_normal((2, *layout, 3, Dh)).astype(np.float32)
        y, tl, post = O.token_permute(x, tile, dil, flip)
        y2 = O.token_permute_by_views(x, tile, dil, flip)
        y3 = _torch_views(torch.from_numpy(x), tile, dil, flip).numpy()
        assert y.shape == y2.shape == y3.shape
        assert (y == y2).all() and (y == y3).all(), (layout, tile, dil, flip)
        assert tl == tuple(layout)
        assert post == tuple(-(-(-(-X // t)) // d) * t for X, t, d in zip(layout, tile, dil))
        back = O.token_unpermute(y, layout, tile, dil, flip)
        assert (back == x).all()


def test_padding_is_zero_and_permutation_is_a_bijection():
    layout, tile, dil = (7, 9, 5), (2, 3, 2), (2, 1, 2)
    src = O.permute_source_coords(layout, tile, dil, True)
    valid = np.all(src < np.array(layout), axis=-1)
    lin = (src[..., 0] * 9 + src[..., 1]) * 5 + src[..., 2]
    assert sorted(lin[valid].tolist()) == list(range(7 * 9 * 5))  # each real token appears exactly once
    x = np.ones((1, *layout, 1, 1))
    y, _, _ = O.token_permute(x, tile, dil, True)
    assert y.sum() == 7 * 9 * 5 and set(np.unique(y)) == {0.0, 1.0}


def test_flip_is_dimension_reversal():
    # flip=True on layout X equals flip=False on the transposed layout with reversed parameters.
    rng = np.random.default_rng(0)
    x = rng.standard_normal((1, 6, 8, 10, 2, 3))
    tile, dil = (2, 4, 5), (3, 1, 2)
    a, _, _ = O.token_permute(x, tile, dil, True)
    xt = np.ascontiguousarray(x.transpose(0, 3, 2, 1, 4, 5))
    b, _, _ = O.token_permute(xt, tile[::-1], dil[::-1], False)
    assert (a == b).all()


def test_dilation_groups_fold_into_batch_group_fastest():
    # batch index of the permuted tensor = b * G + g, g colexicographic over dilation (dim 0 fastest).
    x = np.zeros((3, 4, 6, 1, 1))
    for b in range(3):
        for i in range(4):
            for j in range(6):
                x[b, i, j] = b * 100 + (i % 2) * 10 + (j % 3)
    y, _, _ = O.token_permute(x, (1, 1), (2, 3), True)
    for b in range(3):
        for g in range(6):
            g0, g1 = g % 2, g // 2
            assert (y[b * 6 + g] == b * 100 + g0 * 10 + g1).all()


def test_tiles_are_contiguous_runs_colexicographic():
    # flip=True, no dilation: permuted position p = tile_index * |tile| + offset, both colexicographic.
    layout, tile = (4, 6), (2, 3)
    src = O.permute_source_coords(layout, tile, (1, 1), True)[0]
    for p in range(24):
        ti, off = divmod(p, 6)
        tc = O.idx2crd_colex(ti, (2, 2))
        oc = O.idx2crd_colex(off, tile)
        assert tuple(src[p]) == (tc[0] * 2 + oc[0], tc[1] * 3 + oc[1])
