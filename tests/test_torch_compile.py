"""The public operations under a tracing compiler (torch.compile): the drivers route the native
calls through torch custom operators whose fake implementations give shapes and dtypes, so
the whole call traces into one graph (reference: src/natten/_libnatten/torch_wrappers.py:716-751).

The CPU tests trace with fake device tensors (no GPU is touched); the GPU test runs the
compiled function and compares it with the eager call bit for bit."""

import pytest
import torch
from torch._subclasses.fake_tensor import FakeTensorMode

import natten_amd

CASES = {
    "na2d one launch": (lambda q, k, v: natten_amd.na2d(q, k, v, (5, 5), (1, 1), (1, 1), return_lse=True),
                        [(1, 16, 16, 2, 64)] * 3),
    "na2d permuted": (lambda q, k, v: natten_amd.na2d(q, k, v, (5, 7), (1, 1), (1, 1), return_lse=True),
                      [(1, 20, 24, 2, 64)] * 3),
    "na1d additional kv": (lambda q, k, v, ak, av: natten_amd.na1d(q, k, v, 7, additional_keys=ak, additional_values=av,
                                                                   return_lse=True),
                           [(1, 70, 2, 64)] * 3 + [(1, 13, 2, 64)] * 2),
    "attention": (lambda q, k, v: natten_amd.attention(q, k, v, is_causal=True, return_lse=True), [(2, 100, 4, 32)] * 3),
    "na3d padded head dim": (lambda q, k, v: natten_amd.na3d(q, k, v, (2, 5, 5), return_lse=True),
                             [(1, 4, 8, 8, 2, 40)] * 3),
    "na2d whole-input window": (lambda q, k, v: natten_amd.na2d(q, k, v, (8, 8), return_lse=True), [(1, 8, 8, 2, 64)] * 3),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_traces_into_one_graph_with_fake_tensors(name):
    fn, shapes = CASES[name]
    torch._dynamo.reset()
    with FakeTensorMode():
        args = [torch.empty(s, device="cuda", dtype=torch.bfloat16) for s in shapes]
        compiled = torch.compile(fn, backend="eager", fullgraph=True)
        with torch.no_grad():
            out, lse = compiled(*args)
    assert tuple(out.shape) == tuple(shapes[0]) and out.dtype == torch.bfloat16
    assert tuple(lse.shape) == tuple(shapes[0][:-1]) and lse.dtype == torch.float32


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["na2d one launch", "na2d permuted", "na1d additional kv"])
def test_compiled_equals_eager(name):
    fn, shapes = CASES[name]
    torch._dynamo.reset()
    gen = torch.Generator().manual_seed(0)
    args = [torch.randn(s, generator=gen).to(torch.bfloat16).cuda() for s in shapes]
    with torch.no_grad():
        ref_out, ref_lse = fn(*args)
        out, lse = torch.compile(fn, backend="aot_eager", fullgraph=True)(*args)
    assert torch.equal(out, ref_out) and torch.equal(lse, ref_lse)


def _varlen_attention(q, k, v):
    cu = torch.tensor([0, 40, 170, 300], dtype=torch.int32, device=q.device)
    return natten_amd.attention(q, k, v, is_causal=True, cumulative_seqlen_Q=cu, cumulative_seqlen_KV=cu,
                                max_seqlen_Q=130, max_seqlen_KV=130)


GRAD_CASES = {
    "na2d": (lambda q, k, v: natten_amd.na2d(q, k, v, (5, 7), (2, 1), (1, 1), (False, True)), [(1, 20, 24, 2, 64)] * 3),
    "na3d padded head dim": (lambda q, k, v: natten_amd.na3d(q, k, v, (2, 5, 5)), [(1, 4, 8, 8, 2, 40)] * 3),
    "attention": (lambda q, k, v: natten_amd.attention(q, k, v, is_causal=True), [(2, 100, 4, 32)] * 3),
    # sequence-packed: forward and backward must trace without reading the lengths on the host
    "attention varlen": (_varlen_attention, [(1, 300, 2, 64)] * 3),
}


@pytest.mark.parametrize("name", sorted(GRAD_CASES))
def test_forward_and_backward_trace_with_fake_tensors(name):
    # Inputs that require grad: dynamo has to trace the autograd function's forward *and* backward
    # (it turns both into graphs of custom operators) to compile the call at all.  The backward
    # itself is not run here: the autograd engine wants a real device for "cuda" tensors; the
    # GPU test below runs the compiled training step.
    fn, shapes = GRAD_CASES[name]
    torch._dynamo.reset()
    with FakeTensorMode():
        args = [torch.empty(s, device="cuda", dtype=torch.bfloat16, requires_grad=True) for s in shapes]
        out = torch.compile(fn, backend="eager", fullgraph=True)(*args)
        assert out.requires_grad and out.grad_fn is not None
        assert tuple(out.shape) == tuple(shapes[0]) and out.dtype == torch.bfloat16


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(GRAD_CASES))
def test_compiled_training_step_equals_eager(name):
    fn, shapes = GRAD_CASES[name]
    torch._dynamo.reset()
    gen = torch.Generator().manual_seed(0)
    base = [torch.randn(s, generator=gen).to(torch.bfloat16).cuda() for s in shapes]
    d_out = torch.randn(shapes[0], generator=gen).to(torch.bfloat16).cuda()
    grads = []
    for f in (fn, torch.compile(fn, backend="aot_eager", fullgraph=True)):
        args = [t.clone().requires_grad_(True) for t in base]
        f(*args).backward(d_out)
        grads.append([a.grad for a in args])
    for a, b in zip(*grads):
        assert torch.equal(a, b)
