"""CPU checks of the reference-CPU-path restatement (oracle/flex_cpu.py) and of the two small
copies of the window arithmetic outside the oracle (the tile chooser's and the benchmark's FLOP count).

The mask predicate handed to flex_attention follows the centre-clamp form of the reference's
src/natten/backends/flex.py:333-407; the oracle's mask follows the start / end form of
csrc/include/natten/cuda/reference/mask.hpp:59-91.  They must agree on every (query, key) pair."""

import itertools

import numpy as np
import pytest
import torch

from oracle import na_oracle as O
from oracle.flex_cpu import flex_na_cpu, na_mask_mod

CASES = [
    ((23,), (5,), (2,), (1,), (False,)),
    ((23,), (6,), (3,), (2,), (True,)),
    ((40,), (7,), (7,), (3,), (False,)),
    ((9, 11), (3, 4), (1, 2), (2, 1), (False, True)),
    ((12, 10), (5, 5), (5, 2), (1, 2), (True, False)),
    ((7, 8, 9), (3, 2, 4), (2, 1, 3), (1, 2, 2), (True, False, False)),
    ((6, 6, 10), (6, 3, 5), (1, 3, 4), (1, 1, 2), (False, True, True)),
]


@pytest.mark.parametrize("shape,kernel,stride,dilation,causal", CASES)
def test_mask_mod_equals_oracle_mask(shape, kernel, stride, dilation, causal):
    N = int(np.prod(shape))
    mod = na_mask_mod(shape, kernel, stride, dilation, causal)
    qi = torch.arange(N).view(N, 1).expand(N, N)
    ki = torch.arange(N).view(1, N).expand(N, N)
    got = mod(torch.zeros((), dtype=torch.int64), torch.zeros((), dtype=torch.int64), qi, ki).numpy()
    ref = O.na_mask_dense(shape, kernel, stride, dilation, causal)
    assert got.shape == ref.shape and np.array_equal(got, ref)


def test_mask_mod_random_sweep():
    rng = np.random.default_rng(7)
    for _ in range(60):
        n = int(rng.integers(1, 4))
        shape = tuple(int(rng.integers(4, {1: 60, 2: 14, 3: 8}[n])) for _ in range(n))
        k = tuple(int(rng.integers(2, x + 1)) for x in shape)
        s = tuple(int(rng.integers(1, kk + 1)) for kk in k)
        d = tuple(int(rng.integers(1, x // kk + 1)) for x, kk in zip(shape, k))
        c = tuple(bool(rng.integers(0, 2)) for _ in range(n))
        N = int(np.prod(shape))
        mod = na_mask_mod(shape, k, s, d, c)
        qi = torch.arange(N).view(N, 1).expand(N, N)
        ki = torch.arange(N).view(1, N).expand(N, N)
        got = mod(None, None, qi, ki).numpy()
        assert np.array_equal(got, O.na_mask_dense(shape, k, s, d, c)), (shape, k, s, d, c)


def test_flex_call_matches_dense_oracle_config1():
    # the first benchmark configuration as written: na1d fp32 on CPU, B=1, heads=2, L=256, D=32, k=7, seed 0
    torch.manual_seed(0)
    q, k, v = (torch.randn(1, 256, 2, 32) for _ in range(3))
    out, lse = flex_na_cpu(q, k, v, (7,), (1,), (1,), (False,))
    ref_o, ref_l = O.na_forward(q.numpy(), k.numpy(), v.numpy(), (7,), (1,), (1,), (False,))
    assert np.abs(out.numpy() - ref_o).max() < 1e-4 and np.abs(lse.numpy() - ref_l).max() < 1e-4


def test_flex_call_matches_dense_oracle_2d_gqa():
    torch.manual_seed(1)
    q = torch.randn(2, 10, 12, 4, 16)
    k, v = torch.randn(2, 10, 12, 2, 16), torch.randn(2, 10, 12, 2, 16)
    args = ((5, 4), (2, 3), (2, 1), (True, False))
    out, lse = flex_na_cpu(q, k, v, *args)
    ref_o, ref_l = O.na_forward(q.numpy(), k.numpy(), v.numpy(), *args)
    assert np.abs(out.numpy() - ref_o).max() < 1e-4 and np.abs(lse.numpy() - ref_l).max() < 1e-4


# ---- the window arithmetic outside the oracle ---------------------------------------------------------


def test_tile_chooser_window_equals_oracle_exhaustively():
    from natten_amd.tile_config import _win

    for L in range(2, 34):
        for k in range(2, L + 1):
            for s in range(1, k + 1):
                for causal in (False, True):
                    for i in range(L):
                        st = int(O.window_start(i, k, s, L, causal))
                        en = int(O.window_end(i, st, k, L, causal))
                        assert _win(i, k, s, L, causal) == (st, en), (L, k, s, causal, i)


def test_benchmark_flop_count_equals_oracle():
    import bench

    for L in range(2, 28):
        for k in range(2, L + 1):
            for s in (1, 2, 3, k):
                if s > k:
                    continue
                for d in range(1, L // k + 1):
                    for causal in (False, True):
                        assert bench.count_attended((L,), (k,), (s,), (d,), (causal,)) == \
                            O.count_attended((L,), (k,), (s,), (d,), (causal,)), (L, k, s, d, causal)
    rng = np.random.default_rng(3)
    for _ in range(40):
        n = int(rng.integers(2, 4))
        shape = tuple(int(rng.integers(4, 12)) for _ in range(n))
        k = tuple(int(rng.integers(2, x + 1)) for x in shape)
        s = tuple(int(rng.integers(1, kk + 1)) for kk in k)
        d = tuple(int(rng.integers(1, x // kk + 1)) for x, kk in zip(shape, k))
        c = tuple(bool(rng.integers(0, 2)) for _ in range(n))
        ref = int(O.na_mask_dense(shape, k, s, d, c).sum())
        assert bench.count_attended(shape, k, s, d, c) == ref == O.count_attended(shape, k, s, d, c)
    # the five benchmark configurations (FLOP = 4 B H D x this count)
    for name, flop in (("c2", 2.8353e9), ("c3", 1.3744e11), ("c4", 1.0518e13), ("c5", 1.0995e12)):
        B, H, layout, D, kernel, stride, dilation, causal, _, _ = bench.WORKLOADS[name]
        got = 4.0 * B * H * D * bench.count_attended(layout, kernel, stride, dilation, causal)
        assert abs(got - flop) / flop < 1e-3, (name, got)


def test_traffic_is_only_reported_for_the_current_kernel_sources(tmp_path, monkeypatch):
    import bench

    digest = bench.kernel_digest()
    prof = tmp_path / "profiles"
    prof.mkdir()
    (prof / "x.md").write_text(
        f"traffic: workload=c4 pass=forward q_tile=2,8,8 kv_tile=1,8,8 bytes=1.5e10 kernel_digest={digest}\n"
        "traffic: workload=c3 pass=forward q_tile=8,16 kv_tile=8,8 bytes=7e8 kernel_digest=0123456789abcdef\n")
    monkeypatch.setattr(bench, "ROOT", str(tmp_path))
    monkeypatch.setattr(bench, "kernel_digest", lambda which="forward": digest)
    assert bench.measured_traffic("c4", "forward", (2, 8, 8), (1, 8, 8))["bytes"] == 1.5e10
    assert bench.measured_traffic("c4", "forward", (4, 8, 8), (1, 8, 8)) is None
    assert bench.measured_traffic("c3", "forward", (8, 16), (8, 8)) is None  # measured on other sources


def test_work_queue_default_by_problem_size():
    # the launch kind the ops pick when `run_persistent_kernel` is None: the work queue from 2 048 Q
    # tiles x 32 KV tiles up (every large benchmark shape, causal or not), one workgroup per Q tile below
    import bench
    from natten_amd.functional import _use_work_queue, work_queue_default
    from natten_amd.tile_config import choose_tile_shapes

    expect = {"c1": False, "c2": False, "c2d": False, "c3": False, "c4": True, "c5": True, "hunyuan_na": True,
              "hunyuan_gna": True, "flux_na": True, "flux_gna": True, "odd3d": True,
              "na1d_32k": False, "na1d_32k_s256": False, "na1d_32k_blocked": False}
    for w, (B, H, layout, D, k, s, d, c, _, _) in bench.WORKLOADS.items():
        qt, kt = choose_tile_shapes(layout, k, s, d, c, 128, 64, anchored=True)
        assert work_queue_default(B, H, layout, k, s, d, c, qt, kt) == expect[w], w
    assert _use_work_queue(True, (True,), 1, 1) and not _use_work_queue(False, (False,), 1 << 20, 1 << 10)


def test_every_bench_workload_is_named_and_its_cpu_leg_is_bounded():
    # a workload without a name fails at the end of its run, one whose CPU leg is the full dense
    # problem runs for minutes without output: both are tables that must follow WORKLOADS
    import bench

    for w, (B, H, layout, D, k, s, d, c, _, _) in bench.WORKLOADS.items():
        assert w in bench.WORKLOAD_NAMES, w
        tokens = 1
        for x in layout:
            tokens *= x
        timed = bench.CPU_PROXY[w][0] if w in bench.CPU_PROXY else layout
        n = 1
        for x in timed:
            n *= x
        assert n <= 16384, (w, "dense N x N mask and scores of the CPU leg", n)
        if w in bench.CPU_PROXY:
            # the proxy keeps the window legal: kernel * dilation fits its layout
            assert all(kk * dd <= x for kk, dd, x in zip(k, d, timed)), w
    assert set(bench.REFERENCE_B200_MS) <= set(bench.WORKLOADS)


def test_backward_tile_shapes_per_launch():
    # on the original tensors each backward launch gets the shapes that visit the fewest tiles for its
    # role: the dq launch streams half KV tiles, the dk / dv launch half Q tiles
    from natten_amd.tile_config import _half_tile, choose_backward_role_tile_shapes

    assert _half_tile((2, 8, 8)) == (2, 8, 4) and _half_tile((1, 8, 16)) == (1, 8, 8) and _half_tile((128, 1)) == (64, 1)
    # c4: a causal dimension 0 with one-frame half tiles on the streamed side
    dq, kv = choose_backward_role_tile_shapes((30, 48, 80), (18, 24, 24), (1, 8, 8), (1, 1, 1), (True, False, False))
    assert dq == ((2, 8, 8), (1, 8, 16)) and kv == ((1, 8, 16), (2, 8, 8))
    # shapes need not divide the extents (the kernels move or clamp the tiles at a group's end) ...
    dq, kv = choose_backward_role_tile_shapes((29, 46, 78), (9, 24, 24), (1, 8, 8), (2, 1, 1), (False,) * 3)
    assert dq == ((2, 8, 8), (1, 8, 16)) and kv == ((1, 8, 16), (2, 8, 8))
    # ... but every dilation group must be at least a tile wide in every dimension: none fits here
    assert choose_backward_role_tile_shapes((6, 6), (3, 3), (1, 1), (1, 1), (False, False)) is None
    # 1-D: one factorisation, the same for both launches
    assert choose_backward_role_tile_shapes((4096,), (512,), (1,), (1,), (True,)) == (((128,), (128,)),) * 2
    # whatever is chosen holds 128 tokens and divides the extents
    for layout, k, s, d, c in [((64, 64), (13, 13), (1, 1), (2, 2), (False, False)),
                               ((256, 256), (80, 80), (16, 16), (1, 1), (False, True))]:
        for qt, kt in choose_backward_role_tile_shapes(layout, k, s, d, c):
            for t in (qt, kt):
                p = 1
                for x in t:
                    p *= x
                assert p == 128 and all(X % (dd * x) == 0 for X, dd, x in zip(layout, d, t))
