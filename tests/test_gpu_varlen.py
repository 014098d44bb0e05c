"""GPU parity: variable-length (sequence-packed) dense attention through the public API (C ABI
underneath).  Every sequence is checked against the CPU oracle evaluated on that sequence alone
(atol = rtol = 1e-2), and against the fixed-length entry point called per sequence — the
comparison the reference's tests/test_fmha_varlen.py:216-345 makes.  Sequence lists are those
of tests/test_fmha_varlen.py:722-748 (head dims this build supports) plus edge cases."""

import numpy as np
import pytest
import torch

import natten_amd
from natten_amd.utils.varlen import generate_varlen_parameters
from oracle import na_oracle as O
from tests.gpu_utils import assert_close, to_np

pytestmark = pytest.mark.gpu


def _rand(shape, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=gen).to(dtype).cuda()


def run_varlen(heads, heads_kv, head_dim, seqlens_q, seqlens_kv, causal, dtype, seed, use_cumulative=False,
               oracle_limit=2200):
    tq, tkv = sum(seqlens_q), sum(seqlens_kv)
    q = _rand((1, tq, heads, head_dim), dtype, 3 * seed)
    k = _rand((1, tkv, heads_kv, head_dim), dtype, 3 * seed + 1)
    v = _rand((1, tkv, heads_kv, head_dim), dtype, 3 * seed + 2)
    sq = torch.tensor(seqlens_q, dtype=torch.int32, device="cuda")
    skv = torch.tensor(seqlens_kv, dtype=torch.int32, device="cuda")
    with torch.no_grad():
        if use_cumulative:
            cu_q, cu_kv, mq, mkv = generate_varlen_parameters(q, k, v, sq, skv)
            out, lse = natten_amd.attention(q, k, v, is_causal=causal, return_lse=True, cumulative_seqlen_Q=cu_q,
                                            cumulative_seqlen_KV=cu_kv, max_seqlen_Q=mq, max_seqlen_KV=mkv)
        else:
            out, lse = natten_amd.attention(q, k, v, is_causal=causal, return_lse=True, seqlens_Q=sq, seqlens_KV=skv)
    torch.cuda.synchronize()
    assert out.shape == q.shape and out.dtype == dtype
    assert lse.shape == q.shape[:-1] and lse.dtype == torch.float32
    oq = okv = 0
    for b, (lq, lkv) in enumerate(zip(seqlens_q, seqlens_kv)):
        tag = f"varlen seq {b} of {seqlens_q}/{seqlens_kv} H={heads}/{heads_kv} D={head_dim} causal={causal} {dtype}"
        o_b, l_b = out[:, oq : oq + lq], lse[:, oq : oq + lq]
        if lq > 0 and lkv > 0:
            q_b, k_b, v_b = q[:, oq : oq + lq], k[:, okv : okv + lkv], v[:, okv : okv + lkv]
            with torch.no_grad():
                o_fix, l_fix = natten_amd.attention(q_b.contiguous(), k_b.contiguous(), v_b.contiguous(),
                                                    is_causal=causal, return_lse=True)
            # same arithmetic on the same rows in the same order
            assert torch.equal(o_b, o_fix), "out differs from the fixed-length call: " + tag
            assert torch.equal(l_b, l_fix), "lse differs from the fixed-length call: " + tag
            if lq * lkv <= oracle_limit * oracle_limit:
                ref_o, ref_l = O.attention_forward(to_np(q_b), to_np(k_b), to_np(v_b), is_causal=causal)
                assert_close("out " + tag, to_np(o_b), ref_o)
                assert_close("lse " + tag, to_np(l_b), ref_l)
        elif lq > 0:
            assert torch.count_nonzero(o_b) == 0, "a sequence without keys must give zeros: " + tag
            assert torch.isneginf(l_b).all(), "a sequence without keys must give lse = -inf: " + tag
        oq += lq
        okv += lkv


REFERENCE_PROBLEMS = [
    # heads, head_dim, seqlens_Q, seqlens_KV  (tests/test_fmha_varlen.py:723-748)
    (1, 88, [11, 1846, 2433, 1193], [1681, 2831, 1932, 141]),
    (7, 56, [126, 1127, 3130, 3782, 1445, 751, 594], [746, 2886, 1273, 1399, 33, 3570, 2327]),
    (1, 128, [128, 128, 135, 121, 128, 128], [128, 128, 135, 121, 128, 128]),
    (1, 128, [128, 128, 135, 128, 128], [128, 128, 135, 128, 128]),
    (1, 128, [135, 200], [128, 768]),
    (1, 128, [1024, 200], [128, 768]),
    (1, 128, [135, 200], [135, 768]),
    (1, 128, [1024, 200], [135, 768]),
    (1, 128, [1024, 256], [128, 768]),
    (1, 128, [1024, 8, 17, 2048], [10, 20, 512, 16]),
    (2, 128, [268, 1584, 1571], [2448, 4088, 1925]),
    (1, 128, [1024, 256], [512, 768]),
]


@pytest.mark.parametrize("causal", [False, True])
def test_reference_varlen_problems(causal):
    for i, (heads, head_dim, sq, skv) in enumerate(REFERENCE_PROBLEMS):
        run_varlen(heads, heads, head_dim, sq, skv, causal, torch.float16 if i % 2 else torch.bfloat16, seed=i)


def test_cumulative_arguments_and_gqa():
    run_varlen(4, 2, 64, [5, 300, 64, 1], [70, 1, 129, 64], False, torch.bfloat16, seed=20, use_cumulative=True)
    run_varlen(6, 1, 32, [257, 3], [3, 257], True, torch.float16, seed=21, use_cumulative=True)


def test_single_sequence_equals_plain_attention():
    run_varlen(2, 2, 64, [333], [222], True, torch.bfloat16, seed=30)


def test_empty_sequences():
    # a sequence with no queries, and one with queries but no keys (out = 0, lse = -inf)
    run_varlen(2, 2, 64, [40, 0, 130], [50, 20, 70], False, torch.bfloat16, seed=40)
    run_varlen(2, 1, 128, [40, 17, 130], [50, 0, 70], True, torch.float16, seed=41)


def test_rows_outside_every_sequence_are_zero():
    # cumulative lengths that stop short of the packed tensors: the tail belongs to no sequence
    q, k, v = (_rand((1, 100, 2, 64), torch.bfloat16, s) for s in (1, 2, 3))
    cu = torch.tensor([0, 30, 80], dtype=torch.int32, device="cuda")
    with torch.no_grad():
        out, lse = natten_amd.attention(q, k, v, return_lse=True, cumulative_seqlen_Q=cu, cumulative_seqlen_KV=cu,
                                        max_seqlen_Q=50, max_seqlen_KV=50)
    assert torch.count_nonzero(out[:, 80:]) == 0 and torch.count_nonzero(lse[:, 80:]) == 0
    ref_o, ref_l = O.attention_forward(to_np(q[:, 30:80]), to_np(k[:, 30:80]), to_np(v[:, 30:80]))
    assert_close("out", to_np(out[:, 30:80]), ref_o)
    assert_close("lse", to_np(lse[:, 30:80]), ref_l)


def test_malformed_cumulative_lengths_are_not_followed():
    # cumulative arrays the tensors cannot hold (past the end, decreasing, negative): the kernel
    # leaves the rows of such a sequence untouched (zeros) instead of forming addresses from
    # them; the well-formed sequence in the same launch is computed as usual
    from natten_amd import _lib

    q, k, v = (_rand((1, 100, 2, 64), torch.bfloat16, s) for s in (4, 5, 6))
    good = torch.tensor([0, 40], dtype=torch.int32, device="cuda")
    for bad_tail in ([5000], [-7], [20]):
        cu_q = torch.tensor([0, 40] + bad_tail, dtype=torch.int32, device="cuda")
        cu_kv = torch.tensor([0, 40, 100], dtype=torch.int32, device="cuda")
        for a, b in ((cu_q, cu_kv), (cu_kv, cu_q)):
            out, lse = _lib.attention_forward_varlen(q, k, v, a, b, 60, 60, False, 0.125)
            torch.cuda.synchronize()
            ref_o, ref_l = _lib.attention_forward_varlen(q, k, v, good, good, 60, 60, False, 0.125)
            assert torch.equal(out[:, :40], ref_o[:, :40]) and torch.equal(lse[:, :40], ref_l[:, :40])
            assert torch.count_nonzero(out[:, 40:]) == 0 and torch.count_nonzero(lse[:, 40:]) == 0


@pytest.mark.parametrize("causal", [False, True])
def test_varlen_backward(causal):
    # gradients of the packed call against the backward oracle evaluated per sequence
    seqlens_q, seqlens_kv = [70, 1, 0, 200, 33], [64, 5, 9, 130, 0]
    H, Hkv, D, dtype = 4, 2, 64, torch.bfloat16
    tq, tkv = sum(seqlens_q), sum(seqlens_kv)
    q = _rand((1, tq, H, D), dtype, 50).requires_grad_(True)
    k = _rand((1, tkv, Hkv, D), dtype, 51).requires_grad_(True)
    v = _rand((1, tkv, Hkv, D), dtype, 52).requires_grad_(True)
    d_out = _rand((1, tq, H, D), dtype, 53)
    sq = torch.tensor(seqlens_q, dtype=torch.int32, device="cuda")
    skv = torch.tensor(seqlens_kv, dtype=torch.int32, device="cuda")
    natten_amd.attention(q, k, v, is_causal=causal, seqlens_Q=sq, seqlens_KV=skv).backward(d_out)
    oq = okv = 0
    for lq, lkv in zip(seqlens_q, seqlens_kv):
        if lq > 0 and lkv > 0:
            ref = O.attention_backward(to_np(q[:, oq : oq + lq]), to_np(k[:, okv : okv + lkv]), to_np(v[:, okv : okv + lkv]),
                                       to_np(d_out[:, oq : oq + lq]), is_causal=causal)
            got = (q.grad[:, oq : oq + lq], k.grad[:, okv : okv + lkv], v.grad[:, okv : okv + lkv])
            for name, g, r in zip(("dq", "dk", "dv"), got, ref):
                assert_close(f"{name} seq ({lq},{lkv}) causal={causal}", to_np(g), r, atol=2e-2, rtol=2e-2)
        else:
            assert torch.count_nonzero(q.grad[:, oq : oq + lq]) == 0
            assert torch.count_nonzero(k.grad[:, okv : okv + lkv]) == 0 and torch.count_nonzero(v.grad[:, okv : okv + lkv]) == 0
        oq += lq
        okv += lkv


@pytest.mark.parametrize("head_dim,dtype", [(128, torch.float16), (32, torch.bfloat16)])
def test_varlen_backward_equals_per_sequence_calls(head_dim, dtype):
    # one set of launches for the packed batch gives, bit for bit, what the fixed-length backward
    # gives sequence by sequence (same kernels, same 128-row tiles); lengths span several tiles
    seqlens_q, seqlens_kv = [300, 128, 1, 513], [257, 640, 77, 130]
    H, Hkv = 2, 1
    tq, tkv = sum(seqlens_q), sum(seqlens_kv)
    q = _rand((1, tq, H, head_dim), dtype, 60)
    k = _rand((1, tkv, Hkv, head_dim), dtype, 61)
    v = _rand((1, tkv, Hkv, head_dim), dtype, 62)
    d_out = _rand((1, tq, H, head_dim), dtype, 63)
    sq = torch.tensor(seqlens_q, dtype=torch.int32, device="cuda")
    skv = torch.tensor(seqlens_kv, dtype=torch.int32, device="cuda")
    for causal in (False, True):
        qp, kp, vp = (t.clone().requires_grad_(True) for t in (q, k, v))
        natten_amd.attention(qp, kp, vp, is_causal=causal, seqlens_Q=sq, seqlens_KV=skv).backward(d_out)
        oq = okv = 0
        for lq, lkv in zip(seqlens_q, seqlens_kv):
            qs = q[:, oq : oq + lq].clone().requires_grad_(True)
            ks = k[:, okv : okv + lkv].clone().requires_grad_(True)
            vs = v[:, okv : okv + lkv].clone().requires_grad_(True)
            natten_amd.attention(qs, ks, vs, is_causal=causal).backward(d_out[:, oq : oq + lq])
            assert torch.equal(qp.grad[:, oq : oq + lq], qs.grad), (lq, lkv, causal)
            assert torch.equal(kp.grad[:, okv : okv + lkv], ks.grad), (lq, lkv, causal)
            assert torch.equal(vp.grad[:, okv : okv + lkv], vs.grad), (lq, lkv, causal)
            oq += lq
            okv += lkv


def test_gradients_of_rows_outside_every_sequence_are_zero():
    # cumulative lengths that stop short of the packed tensors, forward and backward
    q, k, v = (_rand((1, 100, 2, 64), torch.bfloat16, s).requires_grad_(True) for s in (1, 2, 3))
    d_out = _rand((1, 100, 2, 64), torch.bfloat16, 4)
    cu = torch.tensor([0, 30, 80], dtype=torch.int32, device="cuda")
    natten_amd.attention(q, k, v, cumulative_seqlen_Q=cu, cumulative_seqlen_KV=cu, max_seqlen_Q=50,
                         max_seqlen_KV=50).backward(d_out)
    for t in (q, k, v):
        assert torch.isfinite(t.grad).all() and torch.count_nonzero(t.grad[:, 80:]) == 0
    ref = O.attention_backward(to_np(q[:, 30:80]), to_np(k[:, 30:80]), to_np(v[:, 30:80]), to_np(d_out[:, 30:80]))
    for name, t, r in zip(("dq", "dk", "dv"), (q, k, v), ref):
        assert_close(name, to_np(t.grad[:, 30:80]), r, atol=2e-2, rtol=2e-2)
