"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol the
header declares, argument validation raises the reference's exception classes, tile choice."""

import ctypes
import os
import re

import numpy as np
import pytest
import torch

import natten_amd
from natten_amd import _lib, checks, tile_config

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "natten_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(natten_amd_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 8
    assert os.path.exists(_lib.LIB_PATH), "libnatten_amd.so is not built (python -m natten_amd.build)"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/natten_amd.h but not exported"
    assert sorted(_lib.EXPORTED_SYMBOLS) == names
    assert lib.natten_amd_abi_version() == _lib.ABI_VERSION


def test_supported_tiles_query_matches_python_table():
    for dt in (torch.float16, torch.bfloat16):
        for d in (32, 64, 128):
            assert _lib.supported_tile_sizes(dt, d) == tile_config.TILE_SIZES
    assert _lib.supported_tile_sizes(torch.float16, 48) == []


def test_argument_normalisation_and_errors():
    assert checks.check_all_args(2, 3, None, None, None) == ((3, 3), (1, 1), (1, 1), (False, False))
    assert checks.check_all_args(3, (3, 4, 5), 2, (1, 2, 3), (True, False, True)) == (
        (3, 4, 5), (2, 2, 2), (1, 2, 3), (True, False, True))
    for bad in (1, (3,), (3, 1), 3.0, "3"):
        with pytest.raises(ValueError):
            checks.check_kernel_size_arg(2, bad)
    with pytest.raises(ValueError):
        checks.check_stride_arg(2, 0)
    with pytest.raises(ValueError):
        checks.check_dilation_arg(1, (1, 1))
    with pytest.raises(ValueError):
        checks.check_causal_arg(2, (True,))
    with pytest.raises(ValueError):
        checks.check_causal_arg(2, 1)


def test_tensor_checks():
    q = torch.zeros(1, 8, 8, 4, 16)
    checks.na_tensor_checks(q, q, q)
    with pytest.raises(ValueError):
        checks.na_tensor_checks(q, q[:, :4], q)  # token layout mismatch
    with pytest.raises(ValueError):
        checks.na_tensor_checks(q, q[..., :3, :], q)  # K and V heads differ
    with pytest.raises(ValueError):
        checks.na_tensor_checks(q, q[..., :3, :], q[..., :3, :])  # 3 does not divide 4
    checks.na_tensor_checks(q, q[..., :2, :], q[..., :2, :])  # GQA
    with pytest.raises(ValueError):
        checks.na_tensor_checks(q, q.half(), q)
    with pytest.raises(ValueError):
        checks.na_tensor_checks(q[0], q[0], q[0])  # rank 4 is fine, rank 3 is not
        checks.na_tensor_checks(q[0, 0], q[0, 0], q[0, 0])
    with pytest.raises(ValueError):
        checks.check_args_against_input(q, (5, 5), (1, 1), (2, 2), (False, False))
    with pytest.raises(ValueError):
        checks.check_args_against_input(q, (3, 3), (4, 1), (1, 1), (False, False))
    with pytest.raises(ValueError):
        checks.additional_kv_tensor_checks(q, q, q, torch.zeros(1, 5, 4, 16), None)


def test_is_self_attention_rules():
    q1 = torch.zeros(1, 16, 2, 8)
    assert checks.is_self_attention(q1, (16,), (True,), False)  # 1-D full window, causal or not
    assert not checks.is_self_attention(q1, (16,), (True,), True)
    assert checks.is_self_attention(q1, (16,), (False,), True)
    q2 = torch.zeros(1, 8, 6, 2, 8)
    assert checks.is_self_attention(q2, (8, 6), (False, False), False)
    assert not checks.is_self_attention(q2, (8, 6), (True, False), False)
    assert not checks.is_self_attention(q2, (8, 5), (False, False), False)


def test_tile_choice_prefers_block_aligned_tiles():
    qt, kt = tile_config.choose_tile_shapes(
        (30, 48, 80), (18, 24, 24), (1, 8, 8), (1, 1, 1), (True, False, False), 128, 64)
    assert qt == (2, 8, 8) and kt == (1, 8, 8)
    q = torch.zeros(1, 16, 16, 1, 32)
    with pytest.raises(ValueError):
        tile_config.check_fna_forward_config(q, (3, 3), (1, 1), (1, 1), (False, False), (16, 8), None)
    with pytest.raises(ValueError):
        tile_config.check_fna_forward_config(q, (3, 3), (1, 1), (1, 1), (False, False), (10, 10), (8, 8))
    assert tile_config.check_fna_forward_config(q, (3, 3), (1, 1), (1, 1), (False, False), (16, 8), (8, 8)) == (
        (16, 8), (8, 8))


def test_cpu_tensors_are_rejected_not_emulated():
    q = torch.zeros(1, 16, 16, 1, 32, dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError):
        natten_amd.na2d(q, q, q, kernel_size=3)
    with pytest.raises(NotImplementedError):
        natten_amd.attention(q.flatten(1, 2), q.flatten(1, 2), q.flatten(1, 2))
    with pytest.raises(RuntimeError):
        natten_amd.token_permute_operation(q, (4, 4))


def test_query_range_matches_brute_force():
    """The interval of queries whose window meets a run of keys (what the dK/dV kernel iterates
    over): the library's bisection against an exhaustive scan with the oracle's window functions."""
    from natten_amd import _lib
    from oracle import na_oracle as O

    rng = np.random.default_rng(5)
    cases = [(L, k, s, c) for L in (1, 2, 7, 16, 33) for k in range(1, L + 1) for s in range(1, k + 1) for c in (False, True)
             if not (k == 1 and L > 1)]
    for L, k, s, c in cases:
        win = [(int(O.window_start(q, k, s, L, c)),) for q in range(L)]
        win = [(st, int(O.window_end(q, st, k, L, c))) for q, (st,) in enumerate(win)]
        for _ in range(6):
            j0 = int(rng.integers(0, L))
            j1 = int(rng.integers(j0, min(L, j0 + 9)))
            hits = [q for q, (st, en) in enumerate(win) if en > j0 and st <= j1]
            first, last = _lib.query_range(j0, j1, k, s, L, L, c)
            if hits:
                assert (first, last) == (hits[0], hits[-1]), (L, k, s, c, j0, j1)
            else:
                assert first > last, (L, k, s, c, j0, j1)


def test_route_predicates_keep_32_bit_tile_offsets():
    # the kernels that gather tiles from the original tensors use 32-bit byte offsets inside a
    # tile: a tile that spans 2^31 bytes or more must take the token-permuted route
    row_bytes = 24 * 128 * 2
    assert _lib.fused_layout_supported((32, 48, 80), (1, 1, 1), (1, 8, 8), row_bytes=row_bytes)
    assert _lib.backward_fused_layout_supported((32, 48, 80), (1, 1, 1), (2, 8, 8), (2, 8, 8), row_bytes=row_bytes)
    # 128 planes of 512 x 512 tokens: a (128, 1, 1) tile spans 127 planes = 204 GB
    big = (128, 512, 512)
    assert _lib.fused_layout_supported(big, (1, 1, 1), (1, 8, 8), row_bytes=row_bytes)
    assert not _lib.fused_layout_supported(big, (1, 1, 1), (64, 1, 1), row_bytes=row_bytes)
    assert not _lib.backward_fused_layout_supported(big, (1, 1, 1), (128, 1, 1), (2, 8, 8), row_bytes=row_bytes)
    assert not _lib.backward_fused_layout_supported(big, (1, 1, 1), (2, 8, 8), (128, 1, 1), row_bytes=row_bytes)
    assert _lib.backward_fused_layout_supported(big, (1, 1, 1), (2, 8, 8), (2, 8, 8), row_bytes=row_bytes)
    # extents that are not multiples of dilation x tile are refused as before
    assert not _lib.fused_layout_supported((20, 24), (1, 1), (8, 8), row_bytes=1024)


def test_backward_entry_point_rejects_tiles_beyond_32_bit_offsets():
    # argument validation happens before anything touches a device: fake (aligned, non-null)
    # pointers are never dereferenced on this path
    import ctypes as C

    L = _lib.lib()
    i32 = lambda xs: (C.c_int32 * 3)(*xs)
    ptr = 0x10000
    rc = L.natten_amd_fna_backward_fused(
        ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, 2 * ptr, _lib.DTYPE_CODES[__import__("torch").bfloat16], 3, 1, 24, 24, 128,
        i32((128, 512, 512)), i32((3, 3, 3)), i32((1, 1, 1)), i32((1, 1, 1)), i32((0, 0, 0)), i32((128, 1, 1)),
        i32((2, 8, 8)), C.c_float(0.1), 3, None,
    )
    assert rc != 0 and b"2^31 bytes" in L.natten_amd_last_error()
    # `roles` names the launches to make: 1 (dq), 2 (dk and dv) or 3
    rc = L.natten_amd_fna_backward_fused(
        ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, 2 * ptr, _lib.DTYPE_CODES[__import__("torch").bfloat16], 3, 1, 24, 24, 128,
        i32((16, 16, 16)), i32((3, 3, 3)), i32((1, 1, 1)), i32((1, 1, 1)), i32((0, 0, 0)), i32((2, 8, 8)),
        i32((2, 8, 8)), C.c_float(0.1), 0, None,
    )
    assert rc != 0 and b"roles" in L.natten_amd_last_error()
    # the dk / dv launch needs the workspace of the scaled queries, which cannot be q itself
    for q_scaled, roles, message in ((None, 2, b"q_scaled workspace"), (None, 3, b"q_scaled workspace"), (ptr, 3, b"must not be q")):
        rc = L.natten_amd_fna_backward_fused(
            ptr, 3 * ptr, 3 * ptr, 3 * ptr, 3 * ptr, 3 * ptr, 3 * ptr, 3 * ptr, 3 * ptr, q_scaled,
            _lib.DTYPE_CODES[__import__("torch").bfloat16], 3, 1, 24, 24, 128, i32((16, 16, 16)), i32((3, 3, 3)),
            i32((1, 1, 1)), i32((1, 1, 1)), i32((0, 0, 0)), i32((2, 8, 8)), i32((2, 8, 8)), C.c_float(0.1), roles, None,
        )
        assert rc != 0 and message in L.natten_amd_last_error(), L.natten_amd_last_error()


def test_every_entry_point_rejects_null_arguments_before_touching_a_device():
    # argument validation comes first in every entry point: all-zero arguments (null pointers,
    # zero sizes) give an error code and a message, without any device call
    import ctypes as C

    L = _lib.lib()
    skipped = {"natten_amd_abi_version", "natten_amd_last_error", "natten_amd_fna_supported_tiles",
               "natten_amd_fna_forward_workspace_bytes"}
    checked = 0
    for name, (_, arg_types) in _lib._SIGNATURES.items():
        if name in skipped:
            continue
        zeros = [None if a is C.c_void_p else (0.0 if a is C.c_float else 0) for a in arg_types]
        rc = getattr(L, name)(*zeros)
        assert rc != 0, f"{name} accepted null arguments"
        assert L.natten_amd_last_error(), f"{name} returned an error without a message"
        checked += 1
    assert checked >= 14


def test_work_queue_launch_needs_a_workspace():
    # run_persistent without a workspace, with one that is too small, or misaligned: refused with
    # a message before any device call (the other arguments are not even looked at)
    import ctypes as C

    L = _lib.lib()
    need = L.natten_amd_fna_forward_workspace_bytes()
    assert need == 512
    for name in ("natten_amd_fna_forward", "natten_amd_fna_forward_fused"):
        arg_types = _lib._SIGNATURES[name][1]
        for ws, nbytes in ((None, 0), (4096, need - 1), (4096 + 32, need)):
            args = [None if a is C.c_void_p else (0.0 if a is C.c_float else 0) for a in arg_types]
            args[6] = 1  # na_dim
            args[-4], args[-3], args[-2] = 1, ws, nbytes
            assert getattr(L, name)(*args) != 0
            assert b"workspace" in L.natten_amd_last_error(), L.natten_amd_last_error()
            args[-4] = 2  # "the workspace is already zero" needs a workspace just the same
            assert getattr(L, name)(*args) != 0
            assert b"workspace" in L.natten_amd_last_error(), L.natten_amd_last_error()
        args[-4], args[-3], args[-2] = 3, 4096, need
        assert getattr(L, name)(*args) != 0
        assert b"run_persistent must be 0, 1 or 2" in L.natten_amd_last_error(), L.natten_amd_last_error()


def test_kernel_window_arithmetic_equals_oracle():
    # natten_amd_window runs the routine of the kernels' set-up (stride division by multiply and
    # shift); against the oracle's window for every query of every small problem, and for large
    # coordinates and strides at random
    from oracle import na_oracle as O

    for L in range(1, 40):
        for k in range(1, L + 1):
            for s in range(1, k + 1):
                for causal in (False, True):
                    for i in range(L + 3):  # queries past the extent (padding) get a window too
                        st = int(O.window_start(i, k, s, L, causal))
                        assert _lib.window(i, k, s, L, causal) == (st, int(O.window_end(i, st, k, L, causal)))
    rng = np.random.default_rng(5)
    for _ in range(3000):
        L = int(rng.integers(1, 2**30))
        k = int(rng.integers(1, L + 1))
        s = int(rng.integers(1, k + 1))
        i = int(rng.integers(0, L))
        causal = bool(rng.integers(0, 2))
        st = int(O.window_start(i, k, s, L, causal))
        assert _lib.window(i, k, s, L, causal) == (st, int(O.window_end(i, st, k, L, causal))), (i, k, s, L, causal)
