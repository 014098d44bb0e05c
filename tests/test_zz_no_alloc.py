"""The entry point that allocates nothing (natten_amd_fna_forward_fused_static: work-queue launch
whose queues live in a static device array of the library) against the existing entry point
(natten_amd_fna_forward_fused with a caller workspace), through the C ABI: bit-equal outputs on
two calls in a row, the second with a smaller input, and both within tolerance of the oracle."""

import pytest
import torch

from natten_amd import _lib
from tests.gpu_utils import assert_close, make_qkv, oracle_full, to_np

pytestmark = pytest.mark.gpu


def _both(shape, H, Hkv, D, dtype, k, s, d, causal, qt, kt, seed):
    q, kk, v = make_qkv(2, shape, H, Hkv, D, dtype, seed=seed)
    scale = D**-0.5
    out = torch.full_like(q, float("nan"))
    lse = torch.full(q.shape[:-1], float("nan"), dtype=torch.float32, device=q.device)
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    _lib.fna_forward_fused_static(q, kk, v, out, lse, k, s, d, causal, scale, qt, kt)
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before  # not even through torch
    torch.cuda.synchronize()
    ref_out, ref_lse = _lib.fna_forward_fused(q, kk, v, k, s, d, causal, scale, qt, kt, run_persistent=True)
    one_out, one_lse = _lib.fna_forward_fused(q, kk, v, k, s, d, causal, scale, qt, kt, run_persistent=False)
    torch.cuda.synchronize()
    assert torch.equal(out, ref_out) and torch.equal(lse, ref_lse)
    assert torch.equal(out, one_out) and torch.equal(lse, one_lse)
    o, l = oracle_full(q, kk, v, k, s, d, causal)
    assert_close("out", to_np(out), o)
    assert_close("lse", to_np(lse), l)


def test_static_scratch_entry_point_two_calls_second_smaller():
    # 3-D, many more Q tiles than resident workgroups would be at full size; then a smaller 2-D problem
    _both((8, 24, 32), 4, 2, 128, torch.bfloat16, (5, 9, 12), (1, 4, 4), (1, 1, 1), (True, False, False), (2, 8, 8),
          (1, 8, 8), seed=21)
    _both((16, 32), 2, 2, 64, torch.float16, (7, 5), (2, 1), (1, 2), (False, False), (8, 16), (8, 8), seed=22)


def test_static_scratch_entry_point_refuses_what_the_work_queue_kernel_does_not_take():
    q, kk, v = make_qkv(1, (16, 32), 2, 2, 64, torch.bfloat16, seed=1)
    out, lse = torch.empty_like(q), torch.empty(q.shape[:-1], dtype=torch.float32, device=q.device)
    with pytest.raises(RuntimeError, match="Q tiles of 128"):
        _lib.fna_forward_fused_static(q, kk, v, out, lse, (5, 5), (1, 1), (1, 1), (False, False), 0.125, (16, 16), (8, 8))
    with pytest.raises(RuntimeError, match="fp16 / bf16"):
        L = _lib.lib()
        q8 = q.to(torch.float8_e4m3fn)
        rc = L.natten_amd_fna_forward_fused_static(
            q8.data_ptr(), q8.data_ptr(), q8.data_ptr(), out.data_ptr(), lse.data_ptr(), _lib.DTYPE_CODES[q8.dtype], 2, 1, 2,
            2, 64, _lib._i32([16, 32]), _lib._i32([5, 5]), _lib._i32([1, 1]), _lib._i32([1, 1]), _lib._i32([0, 0]),
            _lib._i32([8, 16]), _lib._i32([8, 8]), 0.125, None, None, None, None)
        _lib._check(rc)
