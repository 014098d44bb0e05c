"""Pins the oracle's floating-point parts and the tile-level traversal (no GPU).

Special cases reduce to library routines (torch scaled_dot_product_attention, logsumexp), the
tiled traversal is brute-forced against the dense mask, and merge is checked against attention
over concatenated keys.
"""

import itertools

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import na_oracle as O
from tests import problems


def _sdpa(q, k, v, causal=False, scale=None):
    # heads-last [B, S, H, D] float64 -> same
    qt, kt, vt = (torch.from_numpy(np.ascontiguousarray(x)).permute(0, 2, 1, 3) for x in (q, k, v))
    o = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, is_causal=causal, scale=scale)
    return o.permute(0, 2, 1, 3).numpy()


def _rand(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape)


def test_full_window_is_plain_attention():
    for shape in [(12,), (5, 6), (3, 4, 5)]:
        q, k, v = (_rand((2, *shape, 3, 8), s) for s in (1, 2, 3))
        o, lse = O.na_forward(q, k, v, kernel_size=shape)
        N = int(np.prod(shape))
        ref = _sdpa(q.reshape(2, N, 3, 8), k.reshape(2, N, 3, 8), v.reshape(2, N, 3, 8))
        np.testing.assert_allclose(o.reshape(2, N, 3, 8), ref, atol=1e-12)
        s = np.einsum("bqhd,bkhd->bhqk", q.reshape(2, N, 3, 8), k.reshape(2, N, 3, 8)) * 8**-0.5
        ref_lse = torch.logsumexp(torch.from_numpy(s), dim=-1).permute(0, 2, 1).numpy()
        np.testing.assert_allclose(lse.reshape(2, N, 3), ref_lse, atol=1e-12)


def test_1d_causal_full_window_is_causal_attention():
    q, k, v = (_rand((1, 19, 2, 16), s) for s in (4, 5, 6))
    o, _ = O.na_forward(q, k, v, kernel_size=19, is_causal=True)
    np.testing.assert_allclose(o, _sdpa(q, k, v, causal=True), atol=1e-12)


def test_stride_equal_kernel_is_blocked_attention():
    # s == k and X % k == 0, non-causal: every block of k tokens attends exactly itself.
    B, H, D = 1, 2, 8
    q, k, v = (_rand((B, 12, 8, H, D), s) for s in (7, 8, 9))
    o, _ = O.na_forward(q, k, v, kernel_size=(4, 2), stride=(4, 2))

    def blocks(x):  # [B, 12, 8, H, D] -> [B*3*4, 8, H, D]
        return x.reshape(B, 3, 4, 4, 2, H, D).transpose(0, 1, 3, 2, 4, 5, 6).reshape(B * 12, 8, H, D)

    ref = _sdpa(blocks(q), blocks(k), blocks(v))
    np.testing.assert_allclose(blocks(o), ref, atol=1e-12)


def test_dilation_is_na_on_each_subgrid():
    q, k, v = (_rand((1, 12, 9, 2, 4), s) for s in (10, 11, 12))
    d = (3, 2)
    o, lse = O.na_forward(q, k, v, kernel_size=(3, 4), stride=(2, 1), dilation=d, is_causal=(False, True))
    for g0 in range(d[0]):
        for g1 in range(d[1]):
            sl = (slice(None), slice(g0, None, d[0]), slice(g1, None, d[1]))
            os_, ls_ = O.na_forward(q[sl], k[sl], v[sl], kernel_size=(3, 4), stride=(2, 1), is_causal=(False, True),
                                    scale=4**-0.5)
            np.testing.assert_allclose(o[sl], os_, atol=1e-12)
            np.testing.assert_allclose(lse[sl], ls_, atol=1e-12)


def test_gqa_equals_repeated_kv_heads():
    q = _rand((1, 9, 7, 6, 8), 1)
    k, v = _rand((1, 9, 7, 2, 8), 2), _rand((1, 9, 7, 2, 8), 3)
    o, lse = O.na_forward(q, k, v, (3, 5), (1, 2))
    o2, lse2 = O.na_forward(q, np.repeat(k, 3, axis=-2), np.repeat(v, 3, axis=-2), (3, 5), (1, 2))
    np.testing.assert_allclose(o, o2, atol=1e-13)
    np.testing.assert_allclose(lse, lse2, atol=1e-13)


def test_merge_equals_attention_over_concatenated_kv():
    # tests/test_attn_merge.py:51-113 pattern: split KV, attend separately, merge.
    q = _rand((2, 10, 3, 8), 1)
    k, v = _rand((2, 30, 3, 8), 2), _rand((2, 30, 3, 8), 3)
    whole_o, whole_l = O.attention_forward(q, k, v)
    for cuts in [(0, 13, 30), (0, 7, 19, 30), (0, 1, 2, 29, 30)]:
        parts = [O.attention_forward(q, k[:, a:b], v[:, a:b]) for a, b in zip(cuts[:-1], cuts[1:])]
        o, l = O.merge_attentions([p[0] for p in parts], [p[1] for p in parts])
        np.testing.assert_allclose(o, whole_o, atol=1e-12)
        np.testing.assert_allclose(l, whole_l, atol=1e-12)
    (o0, l0), (o1, l1) = O.attention_forward(q, k[:, :11], v[:, :11]), O.attention_forward(q, k[:, 11:], v[:, 11:])
    np.testing.assert_allclose(O.merge_attentions([o0, o1], [l0, l1])[1], np.logaddexp(l0, l1), atol=1e-12)


def test_additional_kv_equals_merge_of_two_attentions():
    q, k, v = (_rand((1, 6, 7, 2, 8), s) for s in (1, 2, 3))
    ak, av = _rand((1, 5, 2, 8), 4), _rand((1, 5, 2, 8), 5)
    o, l = O.na_forward(q, k, v, (3, 3), additional_keys=ak, additional_values=av)
    o_na, l_na = O.na_forward(q, k, v, (3, 3))
    o_x, l_x = O.attention_forward(q.reshape(1, 42, 2, 8), ak, av)
    om, lm = O.merge_attentions([o_na.reshape(1, 42, 2, 8), o_x], [l_na.reshape(1, 42, 2), l_x])
    np.testing.assert_allclose(o.reshape(1, 42, 2, 8), om, atol=1e-12)
    np.testing.assert_allclose(l.reshape(1, 42, 2), lm, atol=1e-12)


def test_causal_attention_is_top_left_aligned():
    q, k, v = _rand((1, 4, 1, 8), 1), _rand((1, 9, 1, 8), 2), _rand((1, 9, 1, 8), 3)
    o, _ = O.attention_forward(q, k, v, is_causal=True)
    for i in range(4):
        oi, _ = O.attention_forward(q[:, i : i + 1], k[:, : i + 1], v[:, : i + 1])
        np.testing.assert_allclose(o[:, i : i + 1], oi, atol=1e-13)


# ---- tiled traversal (the structure the fused kernel follows) ---------------------------------

_SMALL_TILED = [
    # shape, k, s, d, causal, q_tile, kv_tile
    ((40,), (7,), (1,), (1,), (False,), (8,), (4,)),
    ((37,), (8,), (3,), (2,), (True,), (8,), (8,)),
    ((125,), (15,), (1,), (1,), (False,), (16,), (8,)),
    ((17, 16), (3, 8), (1, 2), (1, 1), (False, True), (4, 4), (2, 4)),
    ((19, 29), (8, 8), (1, 1), (2, 3), (True, False), (4, 4), (4, 2)),
    ((13, 11, 9), (3, 4, 3), (2, 3, 3), (1, 1, 1), (False, False, False), (2, 4, 2), (2, 2, 2)),
    ((13, 11, 9), (3, 4, 3), (2, 3, 3), (3, 2, 2), (True, False, True), (2, 2, 4), (1, 2, 4)),
    ((8, 8, 16), (3, 3, 3), (2, 1, 2), (2, 2, 4), (False, True, False), (2, 2, 2), (2, 2, 2)),
    ((12, 16), (8, 8), (4, 8), (1, 1), (False, False), (4, 8), (4, 8)),
]


@pytest.mark.parametrize("case", _SMALL_TILED, ids=[str(c[0]) + str(c[4]) for c in _SMALL_TILED])
def test_tiled_traversal_equals_dense(case):
    shape, k, s, d, c, qt, kt = case
    q, kk, v = (_rand((1, *shape, 2, 8), sd) for sd in (1, 2, 3))
    od, ld = O.na_forward(q, kk, v, k, s, d, c)
    stats = {}
    ot, lt = O.na_forward_via_permute(q, kk, v, k, s, d, c, None, qt, kt, stats)
    np.testing.assert_allclose(ot, od, atol=1e-12)
    np.testing.assert_allclose(lt, ld, atol=1e-12)
    assert stats["empty"] == 0  # every tile of the box holds at least one attended pair


def _tile_element_mask(q_first, q_tile, origin, kv_tile, extent, k, s, c):
    n = len(q_tile)
    qs = [np.arange(q_first[a], q_first[a] + q_tile[a]) for a in range(n)]
    ks = [np.arange(origin[a], origin[a] + kv_tile[a]) for a in range(n)]
    m = None
    for a in range(n):
        st = O.window_start(qs[a], k[a], s[a], extent[a], c[a])
        en = O.window_end(qs[a], st, k[a], extent[a], c[a])
        ma = (ks[a][None, :] >= st[:, None]) & (ks[a][None, :] < en[:, None])  # [tq_a, tk_a]
        m = ma if m is None else (m[:, None, :, None] & ma[None, :, None, :]).reshape(m.shape[0] * ma.shape[0], -1)
    return m


def test_tile_box_and_classifier_brute_force():
    rng = np.random.default_rng(3)
    checked = 0
    for _ in range(60):
        n = int(rng.integers(1, 4))
        extent = tuple(int(rng.integers(4, {1: 24, 2: 11, 3: 7}[n])) for _ in range(n))
        k = tuple(int(rng.integers(2, x + 1)) for x in extent)
        s = tuple(int(rng.integers(1, kk + 1)) for kk in k)
        c = tuple(bool(rng.integers(0, 2)) for _ in range(n))
        qt = tuple(int(rng.choice([1, 2, 4])) for _ in range(n))
        kt = tuple(int(rng.choice([1, 2, 4])) for _ in range(n))
        q_shape = tuple(O.ceil_div(x, t) * t for x, t in zip(extent, qt))
        kv_shape = tuple(O.ceil_div(x, t) * t for x, t in zip(extent, kt))
        q_tiled = tuple(a // b for a, b in zip(q_shape, qt))
        kv_tiled = tuple(a // b for a, b in zip(kv_shape, kt))
        for qti in range(int(np.prod(q_tiled))):
            tc = O.idx2crd_colex(qti, q_tiled)
            q_first = tuple(tc[a] * qt[a] for a in range(n))
            start, ntiles = O.kv_tile_box(qti, q_shape, qt, kt, extent, k, s, c)
            in_box = set()
            for it in range(int(np.prod(ntiles))):
                itc = O.idx2crd_colex(it, ntiles)
                in_box.add(tuple(start[a] // kt[a] + itc[a] for a in range(n)))
            for kvc in itertools.product(*[range(x) for x in kv_tiled]):
                origin = tuple(kvc[a] * kt[a] for a in range(n))
                em = _tile_element_mask(q_first, qt, origin, kt, extent, k, s, c)
                cls = O.classify_tile(q_first, qt, origin, kt, extent, k, s, c)
                if em.any():
                    assert kvc in in_box  # the box never drops a tile that has work
                assert (cls == O.TILE_FULL) == bool(em.all())
                assert (cls == O.TILE_EMPTY) == (not em.any())
                checked += 1
    assert checked > 2000


def test_c_oracle_equals_numpy_oracle():
    rng = np.random.default_rng(0)
    for shape, k, s, d, c, H, Hkv in [
        ((13, 11), (3, 4), (2, 3), (2, 2), (True, False), 4, 2),
        ((29,), (8,), (7,), (3,), (False,), 2, 2),
        ((6, 5, 7), (3, 2, 4), (1, 2, 2), (1, 2, 1), (False, True, False), 2, 1),
    ]:
        q = rng.standard_normal((2, *shape, H, 8), dtype=np.float32)
        kk = rng.standard_normal((2, *shape, Hkv, 8), dtype=np.float32)
        v = rng.standard_normal((2, *shape, Hkv, 8), dtype=np.float32)
        od, ld = O.na_forward(q, kk, v, k, s, d, c)
        oc, lc = c_oracle.na_forward(q, kk, v, k, s, d, c, threads=2)
        np.testing.assert_allclose(oc, od, atol=1e-12)
        np.testing.assert_allclose(lc, ld, atol=1e-12)


def test_reference_problem_list_small_cases_tiled():
    # A slice of the reference's own problem tuples through the tiled traversal (data only).
    picks = [problems.NA_2D[0], problems.NA_2D[3], problems.NA_3D[4], problems.NA_3D[5], problems.NA_3D[6]]
    for (B, H, Hkv, D, shape, k, s, d) in picks:
        n = len(shape)
        rng = np.random.default_rng(1)
        q = rng.standard_normal((1, *shape, 2, 4))
        kk = rng.standard_normal((1, *shape, 1, 4))
        v = rng.standard_normal((1, *shape, 1, 4))
        for c in itertools.product([False, True], repeat=n):
            od, ld = O.na_forward(q, kk, v, k, s, d, c)
            qt = {1: (8,), 2: (4, 4), 3: (2, 2, 4)}[n]
            kt = {1: (4,), 2: (2, 4), 3: (2, 2, 2)}[n]
            ot, lt = O.na_forward_via_permute(q, kk, v, k, s, d, c, None, qt, kt)
            np.testing.assert_allclose(ot, od, atol=1e-12)
            np.testing.assert_allclose(lt, ld, atol=1e-12)
