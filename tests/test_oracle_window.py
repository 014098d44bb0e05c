"""Pins the oracle's integer window math (no GPU).

None of these checks retypes the oracle's formula: they compare two independent formulations,
check closed forms for special cases, and brute-force small cases.
"""

import itertools

import numpy as np
import pytest

from oracle import c_oracle
from oracle import na_oracle as O


def _cases_1d(max_L=24):
    for L in range(2, max_L):
        for k in range(2, L + 1):
            for s in range(1, k + 1):
                for c in (False, True):
                    yield L, k, s, c


def test_two_formulations_agree_1d_exhaustive():
    n = 0
    for L, k, s, c in _cases_1d(22):
        for d in (1, 2, 3):
            if k * d > L:
                continue
            a = O.na_mask_dense((L,), k, s, d, c)
            b = O.window_mask_center_form((L,), k, s, d, c)
            assert (a == b).all(), (L, k, s, c, d)
            n += 1
    assert n > 3000


def test_two_formulations_agree_multidim_random():
    rng = np.random.default_rng(7)
    for _ in range(150):
        n = int(rng.integers(2, 4))
        shape = tuple(int(rng.integers(2, 9 if n == 3 else 14)) for _ in range(n))
        d = tuple(int(rng.integers(1, max(2, x // 2 + 1))) for x in shape)
        k = tuple(int(rng.integers(2, max(3, x // dd + 1))) if x // dd >= 2 else None for x, dd in zip(shape, d))
        if any(v is None for v in k):
            continue
        s = tuple(int(rng.integers(1, kk + 1)) for kk in k)
        c = tuple(bool(rng.integers(0, 2)) for _ in range(n))
        a = O.na_mask_dense(shape, k, s, d, c)
        b = O.window_mask_center_form(shape, k, s, d, c)
        assert (a == b).all(), (shape, k, s, d, c)


def test_noncausal_invariants():
    for L, k, s, c in _cases_1d():
        if c:
            continue
        i = np.arange(L)
        st = O.window_start(i, k, s, L, False)
        en = O.window_end(i, st, k, L, False)
        assert ((en - st) == k).all()  # every query attends exactly k keys
        assert (st >= 0).all() and (en <= L).all()
        leader = np.minimum((i // s) * s + s // 2, L - 1)
        assert ((st <= leader) & (leader < en)).all()  # window contains the group's leader
        assert (np.diff(st) >= 0).all() and (np.diff(en) >= 0).all()  # monotone (tile box relies on it)
        grp = i // s
        for g in np.unique(grp):
            assert len(set(st[grp == g])) == 1  # a stride group shares its window


def test_stride1_is_textbook_clamped_window():
    # stride 1, non-causal: the k nearest keys, shifted (not shrunk) at the borders.
    for L in range(2, 30):
        for k in range(2, L + 1):
            i = np.arange(L)
            expect = np.clip(i - k // 2, 0, L - k)
            assert (O.window_start(i, k, 1, L, False) == expect).all(), (L, k)


def test_causal_invariants():
    for L, k, s, c in _cases_1d():
        if not c:
            continue
        i = np.arange(L)
        st = O.window_start(i, k, s, L, True)
        en = O.window_end(i, st, k, L, True)
        assert (en == i + 1).all()  # window ends at the query itself
        leader = np.minimum((i // s) * s + s - 1, L - 1)
        assert (st == np.maximum(leader - k + 1, 0)).all()
        assert (st <= i).all()  # never empty
        assert (np.diff(st) >= 0).all()
        if s == 1:
            assert ((en - st) == np.minimum(i + 1, k)).all()


def test_dilation_group_extents():
    for X in range(1, 40):
        for d in range(1, X + 1):
            ext = [O.fix_dilation_extent(X, d, g) for g in range(d)]
            assert sum(ext) == X
            assert ext == [len(range(g, X, d)) for g in range(d)]


def test_dilated_mask_is_per_subgrid_mask():
    # With dilation d, group g is the sub-sequence g, g+d, ...; its mask must be the undilated
    # mask of a sequence of that group's length.
    for L, k, s, c, d in [(17, 3, 2, False, 3), (20, 4, 1, True, 2), (11, 2, 2, False, 5), (16, 5, 3, True, 3)]:
        full = O.na_mask_dense((L,), k, s, d, c)
        for g in range(d):
            idx = np.arange(g, L, d)
            sub = full[np.ix_(idx, idx)]
            assert (sub == O.na_mask_dense((len(idx),), k, s, 1, c)).all()
            other = np.setdiff1d(np.arange(L), idx)
            assert not full[np.ix_(idx, other)].any()


def test_multidim_mask_is_product_of_1d_masks():
    shape, k, s, c = (6, 7), (3, 4), (2, 1), (True, False)
    m = O.na_mask_dense(shape, k, s, 1, c).reshape(6, 7, 6, 7)
    m0 = O.na_mask_dense((6,), 3, 2, 1, True)
    m1 = O.na_mask_dense((7,), 4, 1, 1, False)
    assert (m == (m0[:, None, :, None] & m1[None, :, None, :])).all()


def test_count_attended_matches_mask_sum():
    for shape, k, s, d, c in [
        ((9, 8), (3, 4), (2, 3), (2, 1), (True, False)),
        ((30,), (7,), (3,), (2,), (False,)),
        ((5, 6, 7), (2, 3, 3), (1, 2, 3), (2, 1, 2), (False, True, False)),
    ]:
        assert O.count_attended(shape, k, s, d, c) == int(O.na_mask_dense(shape, k, s, d, c).sum())


def test_flop_counts_of_the_five_configs():
    # Closed-form work counts quoted for the benchmark configurations.
    assert O.count_attended((256,), (7,)) == 256 * 7
    assert O.count_attended((64, 64), (13, 13)) == 4096 * 169
    assert O.count_attended((64, 64), (13, 13), 1, (2, 2)) == 4096 * 169
    assert O.count_attended((128, 128), (32, 32), (16, 16)) == 16384 * 1024
    assert O.count_attended((30, 48, 80), (18, 24, 24), (1, 8, 8), 1, (True, False, False)) == 387 * 48 * 80 * 576
    assert O.count_attended((16, 64, 64), (8, 16, 16), (4, 8, 8), (1, 2, 2)) == 65536 * 2048


def test_c_oracle_window_equals_numpy():
    for L, k, s, c in _cases_1d(16):
        for i in range(L):
            st = int(O.window_start(i, k, s, L, c))
            en = int(O.window_end(i, st, k, L, c))
            assert c_oracle.window(i, k, s, L, c) == (st, en)


def test_hand_worked_window_tables():
    # tables derived by hand from the definition (tests/golden/README.md), not by any code
    import json
    import os

    path = os.path.join(os.path.dirname(__file__), "golden", "window_tables.json")
    for c in json.load(open(path))["cases"]:
        L, k, s, causal = c["L"], c["kernel"], c["stride"], c["causal"]
        start = [int(O.window_start(i, k, s, L, causal)) for i in range(L)]
        end = [int(O.window_end(i, start[i], k, L, causal)) for i in range(L)]
        assert start == c["start"], (c, start)
        assert end == c["end"], (c, end)
        # the C oracle and the dense mask agree with the same tables
        mask = O.na_mask_dense((L,), (k,), (s,), (1,), (causal,))
        for i in range(L):
            assert mask[i].nonzero()[0].tolist() == list(range(c["start"][i], c["end"][i]))
