"""Host-side pins of the forward kernels' mask machinery (no GPU): the one-bit-per-key element mask
and the launch-level predicate that selects the instance without mask code."""

from __future__ import annotations

import itertools

import numpy as np
import pytest

from natten_amd import _lib
from natten_amd.tile_config import _factorisations
from oracle import na_oracle as O

pytestmark = pytest.mark.skipif(not _lib.has_lib(), reason="libnatten_amd.so is not built")


def brute_key_mask(tile, lo, hi):
    m = 0
    for i in range(64):
        t0 = i % tile[0]
        t1 = (i // tile[0]) % tile[1]
        t2 = i // (tile[0] * tile[1])
        if all(l <= t < h for t, l, h in zip((t0, t1, t2), lo, hi)):
            m |= 1 << i
    return m


def test_key_mask_every_tile_shape_every_interval():
    # every 64-key tile shape; every interval per dimension for the small extents, a sample for 64
    rng = np.random.default_rng(0)
    for tile in _factorisations(64, 3):
        ranges = []
        for e in tile:
            pairs = [(l, h) for l in range(e + 1) for h in range(e + 1)]  # empty and inverted intervals too
            if len(pairs) > 100:
                pairs = [pairs[i] for i in rng.choice(len(pairs), 100, replace=False)] + [(0, e), (0, 0), (e, e), (1, e - 1)]
            ranges.append(pairs)
        combos = list(itertools.product(*ranges))
        if len(combos) > 4000:
            combos = [combos[i] for i in rng.choice(len(combos), 4000, replace=False)]
        for c in combos:
            lo, hi = [x[0] for x in c], [x[1] for x in c]
            assert _lib.tile_key_mask(tile, lo, hi) == brute_key_mask(tile, lo, hi), (tile, lo, hi)


def test_key_mask_lower_dimensional_tiles():
    assert _lib.tile_key_mask((64,), (3,), (17,)) == brute_key_mask((64, 1, 1), (3, 0, 0), (17, 1, 1))
    assert _lib.tile_key_mask((8, 8), (1, 2), (8, 5)) == brute_key_mask((8, 8, 1), (1, 2, 0), (8, 5, 1))
    assert _lib.tile_key_mask((4, 4, 4), (0, 0, 0), (4, 4, 4)) == (1 << 64) - 1


def brute_fully_block_sparse(shape, k, s, d, c, q_tile, kv_tile, anchored):
    """From the dense mask of every dilation group: every Q tile is whole, all of its queries attend
    the same keys, and those keys are a box of whole KV tiles laid out from the window's first key
    (anchored) or from multiples of the tile extent."""
    n = len(shape)
    for g in itertools.product(*[range(x) for x in d]):
        ext = tuple(O.fix_dilation_extent(X, dd, gg) for X, dd, gg in zip(shape, d, g))
        if any(e % t for e, t in zip(ext, q_tile)):
            return False
        mask = O.na_mask_dense(ext, k, s, 1, c).reshape(*ext, *ext)
        for qt in itertools.product(*[range(e // t) for e, t in zip(ext, q_tile)]):
            sl = tuple(slice(i * t, (i + 1) * t) for i, t in zip(qt, q_tile))
            rows = mask[sl].reshape(-1, *ext)
            if not (rows == rows[0]).all():
                return False
            idx = np.argwhere(rows[0])
            lo, hi = idx.min(0), idx.max(0) + 1
            if int(np.prod(hi - lo)) != len(idx):
                return False  # (a window is always a box; kept as a guard)
            for a in range(n):
                if (hi[a] - lo[a]) % kv_tile[a] or (not anchored and lo[a] % kv_tile[a]):
                    return False
    return True


BLOCK_SPARSE_CASES = [
    # shape, kernel, stride, dilation, causal, q_tile, kv_tile
    ((32, 32), (16, 16), (8, 16), (1, 1), (False, False), (8, 16), (8, 8)),     # the shape family of c3
    ((32, 32), (16, 16), (16, 16), (1, 1), (False, False), (8, 16), (8, 8)),
    ((8, 16, 16), (4, 8, 8), (4, 8, 8), (1, 2, 2), (False, False, False), (2, 8, 8), (2, 4, 8)),  # c5's family
    ((4, 16, 16), (4, 8, 8), (4, 8, 8), (1, 1, 1), (False, False, False), (2, 8, 8), (1, 8, 8)),
    ((256,), (128,), (128,), (1,), (False,), (128,), (64,)),                      # blocked 1-D
    ((512,), (256,), (128,), (1,), (False,), (128,), (64,)),
]
NOT_BLOCK_SPARSE_CASES = [
    ((32, 32), (16, 16), (1, 1), (1, 1), (False, False), (8, 16), (8, 8)),       # stride 1
    ((32, 32), (16, 16), (8, 8), (1, 1), (True, False), (8, 16), (8, 8)),        # a causal dimension
    ((32, 32), (16, 16), (8, 8), (1, 1), (False, False), (16, 8), (8, 8)),       # Q tile spans two stride groups
    ((36, 32), (16, 16), (8, 8), (1, 1), (False, False), (8, 16), (8, 8)),       # extent no tile divides
    ((32, 32), (12, 16), (4, 8), (1, 1), (False, False), (8, 16), (8, 8)),       # window not a multiple of the KV tile
    ((33, 32), (16, 16), (8, 8), (2, 1), (False, False), (8, 16), (8, 8)),       # uneven dilation groups
]


@pytest.mark.parametrize("case", BLOCK_SPARSE_CASES)
def test_predicate_true_on_block_sparse_problems(case):
    shape, k, s, d, c, qt, kt = case
    assert brute_fully_block_sparse(shape, k, s, d, c, qt, kt, True)
    assert _lib.fully_block_sparse(shape, k, s, d, c, qt, kt, True)


@pytest.mark.parametrize("case", NOT_BLOCK_SPARSE_CASES)
def test_predicate_false_on_masked_problems(case):
    shape, k, s, d, c, qt, kt = case
    assert not brute_fully_block_sparse(shape, k, s, d, c, qt, kt, True)
    assert not _lib.fully_block_sparse(shape, k, s, d, c, qt, kt, True)


def test_predicate_never_claims_full_when_the_mask_has_a_hole():
    # random small problems: the predicate may be conservative, never optimistic
    rng = np.random.default_rng(3)
    agree = claimed = 0
    for _ in range(400):
        n = int(rng.integers(1, 3))
        q_tile = _factorisations(128, n)[int(rng.integers(0, len(_factorisations(128, n))))]
        kv_tile = _factorisations(64, n)[int(rng.integers(0, len(_factorisations(64, n))))]
        d = tuple(int(rng.integers(1, 3)) for _ in range(n))
        shape, k, s = [], [], []
        for a in range(n):
            mult = int(rng.integers(1, 4))
            X = q_tile[a] * mult * d[a] + (int(rng.integers(0, 3)) if rng.random() < 0.2 else 0)
            ext = X // d[a]
            kk = int(rng.integers(2, ext + 1)) if ext >= 2 else None
            if kk is None:
                break
            if rng.random() < 0.6:  # windows and strides that favour block sparsity
                kk = max(2, min(ext, kv_tile[a] * int(rng.integers(1, 4))))
            ss = int(rng.integers(1, kk + 1))
            if rng.random() < 0.6:
                ss = min(kk, max(1, q_tile[a] * int(rng.integers(1, 3))))
            shape.append(X); k.append(kk); s.append(ss)
        else:
            if int(np.prod(shape)) > 4096:
                continue
            c = tuple(bool(rng.random() < 0.15) for _ in range(n))
            anchored = bool(rng.integers(0, 2))
            try:
                got = _lib.fully_block_sparse(shape, k, s, d, c, q_tile, kv_tile, anchored)
            except RuntimeError:
                continue  # a geometry the one-launch route does not take
            want = brute_fully_block_sparse(tuple(shape), tuple(k), tuple(s), d, c, q_tile, kv_tile, anchored)
            assert not (got and not want), (shape, k, s, d, c, q_tile, kv_tile, anchored)
            agree += got == want
            claimed += got
    assert claimed > 5 and agree > 300


def _masked_pairs(shape, k, s, c, q_tile, kv_tile, box):
    """(wave box, KV tile) pairs that need the element mask, counted pair by pair from the dense
    per-dimension windows: a tile needs none when every query of the box attends all of it (and it
    lies inside the extent) or no query of the box attends any of it.  Dilation 1, KV tiles laid out
    from the first key of each Q tile's window."""
    n = len(shape)
    start = [[int(O.window_start(i, k[a], s[a], shape[a], c[a])) for i in range(shape[a])] for a in range(n)]
    end = [[int(O.window_end(i, start[a][i], k[a], shape[a], c[a])) for i in range(shape[a])] for a in range(n)]
    count = 0
    for qt in itertools.product(*[range(0, shape[a], q_tile[a]) for a in range(n)]):
        org, tiles = [], []
        for a in range(n):
            last = min(qt[a] + q_tile[a] - 1, shape[a] - 1)
            o = start[a][qt[a]] if shape[a] >= kv_tile[a] else (start[a][qt[a]] // kv_tile[a]) * kv_tile[a]
            org.append(o)
            tiles.append(-(-(end[a][last] - o) // kv_tile[a]))
        for b in itertools.product(*[range(0, q_tile[a], box[a]) for a in range(n)]):
            qs = [range(min(qt[a] + b[a], shape[a] - 1), min(qt[a] + b[a] + box[a] - 1, shape[a] - 1) + 1) for a in range(n)]
            for t in itertools.product(*[range(x) for x in tiles]):
                full, some = True, True
                for a in range(n):
                    o, e = org[a] + t[a] * kv_tile[a], org[a] + (t[a] + 1) * kv_tile[a]
                    inside = all(start[a][i] <= o and e <= end[a][i] for i in qs[a]) and e <= shape[a]
                    touched = any(start[a][i] < e and o < end[a][i] for i in qs[a])
                    full, some = full and inside, some and touched
                count += int(some and not full)
    return count


@pytest.mark.parametrize("case", [
    # shape, kernel, stride, causal, Q tile, KV tile
    ((48, 64), (20, 20), (1, 1), (False, False), (8, 16), (8, 8)),
    ((40, 48), (9, 17), (1, 1), (True, False), (16, 8), (4, 16)),
    ((12, 24, 32), (6, 8, 12), (1, 1, 1), (False, False, False), (2, 8, 8), (2, 4, 8)),
    ((10, 16, 24), (4, 8, 8), (1, 8, 8), (True, False, False), (2, 8, 8), (1, 8, 8)),
    ((16, 16, 16), (5, 5, 5), (1, 2, 1), (False, True, False), (4, 4, 8), (4, 4, 4)),
])
def test_wave_box_has_the_fewest_masked_pairs(case):
    shape, k, s, c, q_tile, kv_tile = case
    n = len(shape)
    got = _lib.wave_box(shape, k, s, (1,) * n, c, q_tile, kv_tile)
    assert int(np.prod(got)) == 32 and all(q % b == 0 for q, b in zip(q_tile, got)), got
    candidates = [b for b in itertools.product(*[[1 << i for i in range(6) if (1 << i) <= q] for q in q_tile])
                  if int(np.prod(b)) == 32]
    counts = {b: _masked_pairs(shape, k, s, c, q_tile, kv_tile, b) for b in candidates}
    assert counts[got] == min(counts.values()), (got, counts)


def test_wave_box_defaults():
    # sequence order (as much of the last dimension as fits) where nothing is gained, e.g. block-sparse shapes
    assert _lib.wave_box((128, 128), (32, 32), (16, 16), (1, 1), (False, False), (8, 16), (8, 8)) == (2, 16)
    assert _lib.wave_box((32768,), (2048,), (1,), (1,), (False,), (128,), (64,)) == (32,)


def test_wave_box_choice_is_cheap_on_the_host():
    # the choice runs inside every forward call: a long sequence (one candidate box: nothing to
    # count) and a large image (counted in closed form per Q tile and box) must cost microseconds
    import time

    t0 = time.perf_counter()
    assert _lib.wave_box((1 << 20,), (1 << 19,), (1,), (1,), (False,), (128,), (64,)) == (32,)
    box = _lib.wave_box((4096, 4096), (255, 255), (1, 1), (1, 1), (False, True), (8, 16), (8, 8))
    assert int(np.prod(box)) == 32
    assert time.perf_counter() - t0 < 0.05
