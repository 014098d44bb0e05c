"""Pins the backward oracles (test infrastructure) without the reference:

* the numpy oracle's closed-form gradients against torch autograd differentiating a dense masked
  softmax(QK^T)V in float64 (autograd derives the gradient itself; it shares no formula with
  the oracle), over 1-D / 2-D / 3-D problems with stride, dilation, causal dims and GQA;
* against central finite differences of the scalar loss on a tiny problem;
* the full-window non-causal case against torch's scaled_dot_product_attention backward;
* the C oracle (window walk, no dense mask) against the numpy oracle.
A dropped `scale`, a missing delta term, dK/dV accumulated over the wrong head group or a
transposed dS each fail at least one of these."""

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import na_oracle as O

CASES = [
    # shape, k, s, d, causal, H, Hkv, D
    ((17,), (5,), (1,), (1,), (False,), 2, 2, 8),
    ((23,), (7,), (3,), (2,), (True,), 4, 2, 8),
    ((16,), (16,), (1,), (1,), (True,), 2, 1, 4),
    ((6, 9), (3, 4), (1, 2), (1, 1), (False, False), 2, 1, 8),
    ((8, 10), (3, 5), (2, 1), (2, 1), (True, False), 3, 3, 4),
    ((4, 5, 6), (2, 3, 3), (1, 1, 2), (1, 1, 2), (True, False, False), 2, 2, 4),
    ((5, 4, 4), (5, 4, 4), (1, 1, 1), (1, 1, 1), (False, False, False), 2, 1, 8),
]


def _inputs(shape, H, Hkv, D, seed, batch=2):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((batch, *shape, H, D)).astype(np.float32)
    k = rng.standard_normal((batch, *shape, Hkv, D)).astype(np.float32)
    v = rng.standard_normal((batch, *shape, Hkv, D)).astype(np.float32)
    do = rng.standard_normal((batch, *shape, H, D)).astype(np.float32)
    return q, k, v, do


def _autograd(q, k, v, do, mask, scale):
    B, H, D = q.shape[0], q.shape[-2], q.shape[-1]
    Hkv = k.shape[-2]
    N = int(np.prod(q.shape[1:-2]))
    tq, tk, tv = (torch.tensor(x.reshape(B, N, x.shape[-2], D), dtype=torch.float64, requires_grad=True) for x in (q, k, v))
    kk = tk.repeat_interleave(H // Hkv, dim=2)
    vv = tv.repeat_interleave(H // Hkv, dim=2)
    s = torch.einsum("bqhd,bkhd->bhqk", tq, kk) * scale
    s = s.masked_fill(~torch.tensor(mask)[None, None], float("-inf"))
    out = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(s, dim=-1), vv)
    out.backward(torch.tensor(do.reshape(B, N, H, D), dtype=torch.float64))
    return tuple(t.grad.numpy().reshape(x.shape) for t, x in ((tq, q), (tk, k), (tv, v)))


@pytest.mark.parametrize("case", range(len(CASES)))
def test_numpy_backward_matches_autograd_of_dense_masked_softmax(case):
    shape, ks, st, dl, ca, H, Hkv, D = CASES[case]
    q, k, v, do = _inputs(shape, H, Hkv, D, case)
    scale = 0.37
    got = O.na_backward(q, k, v, do, ks, st, dl, ca, scale=scale)
    ref = _autograd(q, k, v, do, O.na_mask_dense(shape, ks, st, dl, ca), scale)
    for name, g, r in zip(("dq", "dk", "dv"), got, ref):
        np.testing.assert_allclose(g, r, rtol=1e-9, atol=1e-11, err_msg=f"{name} case {CASES[case]}")


@pytest.mark.parametrize("case", range(len(CASES)))
def test_c_backward_matches_numpy(case):
    shape, ks, st, dl, ca, H, Hkv, D = CASES[case]
    q, k, v, do = _inputs(shape, H, Hkv, D, 100 + case)
    got = c_oracle.na_backward(q, k, v, do, ks, st, dl, ca, scale=None, threads=3)
    ref = O.na_backward(q, k, v, do, ks, st, dl, ca)
    for name, g, r in zip(("dq", "dk", "dv"), got, ref):
        np.testing.assert_allclose(g, r, rtol=1e-9, atol=1e-11, err_msg=f"{name} case {CASES[case]}")


def test_finite_differences():
    shape, ks, st, dl, ca = (7,), (3,), (2,), (1,), (True,)
    q, k, v, do = (x.astype(np.float64) for x in _inputs(shape, 2, 1, 4, 7, batch=1))
    dq, dk, dv = O.na_backward(q, k, v, do, ks, st, dl, ca)

    def loss(q_, k_, v_):
        return float((O.na_forward(q_, k_, v_, ks, st, dl, ca)[0] * do).sum())

    eps = 1e-6
    rng = np.random.default_rng(0)
    for arr, grad, which in ((q, dq, 0), (k, dk, 1), (v, dv, 2)):
        for _ in range(6):
            idx = tuple(int(rng.integers(0, n)) for n in arr.shape)
            args_p, args_m = [q.copy(), k.copy(), v.copy()], [q.copy(), k.copy(), v.copy()]
            args_p[which][idx] += eps
            args_m[which][idx] -= eps
            fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(fd - grad[idx]) < 1e-6 * max(1.0, abs(fd)), (which, idx, fd, grad[idx])


def test_full_window_reduces_to_sdpa_backward():
    shape = (4, 6)
    q, k, v, do = _inputs(shape, 2, 2, 8, 11, batch=1)
    got = O.na_backward(q, k, v, do, shape, 1, 1, False)
    tq, tk, tv = (torch.tensor(x.reshape(1, 24, 2, 8).transpose(0, 2, 1, 3), dtype=torch.float64, requires_grad=True)
                  for x in (q, k, v))
    out = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv)
    out.backward(torch.tensor(do.reshape(1, 24, 2, 8).transpose(0, 2, 1, 3), dtype=torch.float64))
    for g, t in zip(got, (tq, tk, tv)):
        np.testing.assert_allclose(g.reshape(1, 24, 2, 8), t.grad.numpy().transpose(0, 2, 1, 3), rtol=1e-8, atol=1e-10)


def test_dense_attention_backward_causal_cross_lengths():
    # top-left causal mask with more queries than keys
    rng = np.random.default_rng(3)
    q = rng.standard_normal((1, 9, 2, 4))
    k = rng.standard_normal((1, 5, 1, 4))
    v = rng.standard_normal((1, 5, 1, 4))
    do = rng.standard_normal((1, 9, 2, 4))
    got = O.attention_backward(q, k, v, do, is_causal=True, scale=0.5)
    mask = np.arange(9)[:, None] >= np.arange(5)[None, :]
    tq, tk, tv = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (q, k, v))
    s = torch.einsum("bqhd,bkhd->bhqk", tq, tk.repeat_interleave(2, dim=2)) * 0.5
    s = s.masked_fill(~torch.tensor(mask)[None, None], float("-inf"))
    out = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(s, dim=-1), tv.repeat_interleave(2, dim=2))
    out.backward(torch.tensor(do))
    for g, t in zip(got, (tq, tk, tv)):
        np.testing.assert_allclose(g, t.grad.numpy(), rtol=1e-9, atol=1e-11)


@pytest.mark.parametrize("case", [
    # shape, kernel, stride, dilation, causal, H, Hkv
    ((37,), (7,), (2,), (3,), (False,), 2, 1),
    ((9, 14), (3, 5), (1, 2), (2, 1), (True, False), 4, 2),
    ((5, 6, 9), (2, 3, 4), (1, 2, 1), (1, 1, 2), (False, True, False), 2, 2),
])
def test_sampled_backward_checker_agrees_with_the_whole_tensor_oracle(case):
    # The GPU tests of the largest problems check gradients position by position with
    # gpu_utils.sampled_backward_check; here that checker is held against the whole-tensor float64
    # oracle on small problems (every dilation group, stride groups, causal dims, GQA): exact
    # gradients must pass at 1e-9, and a gradient with one perturbed row must fail.
    from tests.gpu_utils import sampled_backward_check

    shape, k, s, d, causal, H, Hkv = case
    D, B = 8, 2
    rng = np.random.default_rng(5)
    q = rng.standard_normal((B, *shape, H, D)).astype(np.float32)
    kk = rng.standard_normal((B, *shape, Hkv, D)).astype(np.float32)
    v = rng.standard_normal((B, *shape, Hkv, D)).astype(np.float32)
    do = rng.standard_normal(q.shape).astype(np.float32)
    out, lse = O.na_forward(q, kk, v, k, s, d, causal)
    dq, dk, dv = O.na_backward(q, kk, v, do, k, s, d, causal)
    t = lambda x: torch.from_numpy(np.ascontiguousarray(x, dtype=np.float64))
    n_tok = int(np.prod(shape))
    args = (t(q), t(kk), t(v), t(do), t(out), t(lse), t(dq), t(dk), t(dv), k, s, d, causal)
    sampled_backward_check(*args, n_samples=2 * n_tok, seed=1, atol=1e-9, rtol=1e-9)
    for which in (6, 7, 8):
        bad = list(args)
        g = args[which].clone()
        g.view(B, n_tok, -1)[1, n_tok // 2] += 1e-3   # the checker samples 2 * n_tok positions: every one is hit
        bad[which] = g
        with pytest.raises(AssertionError):
            sampled_backward_check(*bad, n_samples=4 * n_tok, seed=1, atol=1e-9, rtol=1e-9)
