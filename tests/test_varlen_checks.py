"""Argument rules of variable-length attention (CPU): the checks restate the reference's
src/natten/utils/checks.py:569-726 and src/natten/utils/varlen.py:33-132 — same conditions, same
exception classes, same return convention."""

import pytest
import torch

from natten_amd.utils.varlen import generate_varlen_parameters, varlen_tensor_checks


def _qkv(total_q=10, total_kv=12, batch=1):
    q = torch.zeros(batch, total_q, 2, 8)
    k = torch.zeros(batch, total_kv, 2, 8)
    return q, k, k.clone()


def _i32(*xs):
    return torch.tensor(xs, dtype=torch.int32)


def test_not_varlen_returns_none():
    q, k, v = _qkv()
    assert varlen_tensor_checks(q, k, v) == (None, None, 0, 0)
    assert varlen_tensor_checks(q, k, v, max_seqlen_Q=0, max_seqlen_KV=0) == (None, None, 0, 0)
    assert generate_varlen_parameters(q, k, v) == (None, None, 0, 0)


def test_generate_from_seqlens():
    q, k, v = _qkv()
    cu_q, cu_kv, mq, mkv = generate_varlen_parameters(q, k, v, _i32(3, 0, 7), _i32(5, 6, 1))
    assert cu_q.dtype == torch.int32 and cu_kv.dtype == torch.int32
    assert cu_q.tolist() == [0, 3, 3, 10] and cu_kv.tolist() == [0, 5, 11, 12]
    assert (mq, mkv) == (7, 6) and isinstance(mq, int) and isinstance(mkv, int)
    # the checks route seqlens through the same function
    out = varlen_tensor_checks(q, k, v, seqlens_Q=_i32(3, 0, 7), seqlens_KV=_i32(5, 6, 1))
    assert out[0].tolist() == [0, 3, 3, 10] and out[2:] == (7, 6)


@pytest.mark.parametrize(
    "kwargs",
    [
        dict(seqlens_Q=_i32(10)),                                         # only one of the pair
        dict(seqlens_Q=_i32(10).long(), seqlens_KV=_i32(12)),             # wrong dtype
        dict(seqlens_Q=_i32(10).reshape(1, 1), seqlens_KV=_i32(12)),      # wrong rank
        dict(seqlens_Q=_i32(5, 5), seqlens_KV=_i32(12)),                  # sizes differ
        dict(seqlens_Q=_i32(), seqlens_KV=_i32()),                        # empty
        dict(seqlens_Q=[10], seqlens_KV=[12]),                            # not tensors
        dict(cumulative_seqlen_Q=_i32(0, 10), cumulative_seqlen_KV=_i32(0, 12)),                     # maxima missing
        dict(cumulative_seqlen_Q=_i32(0, 10), cumulative_seqlen_KV=_i32(0, 12), max_seqlen_Q=10.0, max_seqlen_KV=12),
        dict(cumulative_seqlen_Q=_i32(0, 10), cumulative_seqlen_KV=_i32(0, 12), max_seqlen_Q=11, max_seqlen_KV=12),
        dict(cumulative_seqlen_Q=_i32(0, 10), cumulative_seqlen_KV=_i32(0, 12), max_seqlen_Q=10, max_seqlen_KV=13),
        dict(cumulative_seqlen_Q=_i32(0, 10), cumulative_seqlen_KV=_i32(0, 12), max_seqlen_Q=0, max_seqlen_KV=12),
        dict(cumulative_seqlen_Q=_i32(0, 10), cumulative_seqlen_KV=_i32(0, 12), max_seqlen_Q=-1, max_seqlen_KV=-1),
        dict(cumulative_seqlen_Q=[0, 10], cumulative_seqlen_KV=[0, 12], max_seqlen_Q=10, max_seqlen_KV=12),
        dict(cumulative_seqlen_Q=_i32(0, 10).long(), cumulative_seqlen_KV=_i32(0, 12), max_seqlen_Q=10, max_seqlen_KV=12),
        dict(cumulative_seqlen_Q=_i32(0, 10).reshape(1, 2), cumulative_seqlen_KV=_i32(0, 12), max_seqlen_Q=10, max_seqlen_KV=12),
        dict(cumulative_seqlen_Q=_i32(0, 4, 10), cumulative_seqlen_KV=_i32(0, 12), max_seqlen_Q=10, max_seqlen_KV=12),
        dict(cumulative_seqlen_Q=_i32(0), cumulative_seqlen_KV=_i32(0), max_seqlen_Q=10, max_seqlen_KV=12),
    ],
)
def test_invalid_arguments_raise_value_error(kwargs):
    q, k, v = _qkv()
    with pytest.raises(ValueError):
        varlen_tensor_checks(q, k, v, **kwargs)


def test_batch_rules():
    q, k, v = _qkv(batch=2)
    with pytest.raises(ValueError):  # sequence-packed layout only
        varlen_tensor_checks(q, k, v, seqlens_Q=_i32(10), seqlens_KV=_i32(12))
    with pytest.raises(ValueError):
        varlen_tensor_checks(q, k, v, cumulative_seqlen_Q=_i32(0, 10), cumulative_seqlen_KV=_i32(0, 12),
                             max_seqlen_Q=10, max_seqlen_KV=12)
    q1, k1, v1 = _qkv(batch=1)
    with pytest.raises(ValueError):  # batch sizes of q, k, v must agree
        varlen_tensor_checks(q, k1, v1)


def test_valid_cumulative_arguments_pass_through():
    q, k, v = _qkv()
    cu_q, cu_kv = _i32(0, 4, 10), _i32(0, 7, 12)
    out = varlen_tensor_checks(q, k, v, cumulative_seqlen_Q=cu_q, cumulative_seqlen_KV=cu_kv, max_seqlen_Q=6,
                               max_seqlen_KV=7)
    assert out[0] is cu_q and out[1] is cu_kv and out[2:] == (6, 7)
