"""The forward, and a whole training step, under HIP graph capture: the entry points allocate nothing and launch on the
caller's stream, so a captured call replays correctly.  Each replay (with new inputs copied into
the captured tensors, and eager work and synchronisations in between) is compared with the
eager result bit for bit."""

import pytest
import torch

import natten_amd

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,kernel,causal", [((16, 16), (5, 5), (False, True)),   # one launch on the original tensors
                                                 ((20, 24), (5, 7), (False, False))])  # permute + kernel + unpermute
def test_forward_replays_from_a_graph(shape, kernel, causal):
    gen = torch.Generator().manual_seed(0)
    mk = lambda: torch.randn((1, *shape, 2, 64), generator=gen).to(torch.bfloat16).cuda()
    q, k, v = mk(), mk(), mk()
    fn = lambda: natten_amd.na2d(q, k, v, kernel, is_causal=causal, return_lse=True)
    side = torch.cuda.Stream()
    with torch.no_grad():
        with torch.cuda.stream(side):
            for _ in range(2):  # warm-up outside the capture
                fn()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out, lse = fn()
        for i in range(3):
            for t in (q, k, v):
                t.copy_(mk())
            graph.replay()
            torch.cuda.synchronize()
            ref_out, ref_lse = fn()   # eager work between the replays
            torch.cuda.synchronize()
            assert torch.equal(out, ref_out) and torch.equal(lse, ref_lse), f"replay {i} differs from the eager call"


def test_static_entry_point_replays_from_a_graph():
    # the entry point that allocates nothing, captured after one eager call on the device (which
    # resolves the address of the library's static queue array outside any capture)
    from natten_amd import _lib

    shape, kernel, stride, dil, causal, qt, kt = (16, 32), (7, 5), (2, 1), (1, 2), (False, True), (8, 16), (8, 8)
    gen = torch.Generator().manual_seed(5)
    mk = lambda: torch.randn((2, *shape, 2, 64), generator=gen).to(torch.float16).cuda()
    q, k, v = mk(), mk(), mk()
    out = torch.empty_like(q)
    lse = torch.empty(q.shape[:-1], dtype=torch.float32, device=q.device)
    fn = lambda: _lib.fna_forward_fused_static(q, k, v, out, lse, kernel, stride, dil, causal, 0.125, qt, kt)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        fn()  # eager warm-up: first call on this device
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
    for i in range(3):
        for t in (q, k, v):
            t.copy_(mk())
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        ref_out, ref_lse = _lib.fna_forward_fused(q, k, v, kernel, stride, dil, causal, 0.125, qt, kt)  # eager work in between
        torch.cuda.synchronize()
        assert torch.equal(out, ref_out) and torch.equal(lse, ref_lse), f"replay {i} differs from the eager call"


def test_split_forward_replays_from_a_graph():
    # a small grid with long windows: the op splits the KV tiles of every Q tile over several
    # workgroups and merges the partial results -- two launches and two allocations inside the capture
    from natten_amd.functional import kv_splits_default
    from natten_amd.tile_config import check_fna_forward_config

    shape, kernel = (2048,), (1024,)
    gen = torch.Generator().manual_seed(3)
    mk = lambda: torch.randn((1, *shape, 2, 128), generator=gen).to(torch.float16).cuda()
    q, k, v = mk(), mk(), mk()
    qt, kt = check_fna_forward_config(q, kernel, (1,), (1,), (False,), None, None)
    assert kv_splits_default(1, 2, shape, kernel, (1,), (1,), (False,), qt, kt) > 1
    fn = lambda: natten_amd.na1d(q, k, v, kernel, return_lse=True)
    side = torch.cuda.Stream()
    with torch.no_grad():
        with torch.cuda.stream(side):
            for _ in range(2):
                fn()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out, lse = fn()
        for i in range(3):
            for t in (q, k, v):
                t.copy_(mk())
            graph.replay()
            torch.cuda.synchronize()
            ref_out, ref_lse = fn()
            torch.cuda.synchronize()
            assert torch.equal(out, ref_out) and torch.equal(lse, ref_lse), f"replay {i} differs from the eager call"


@pytest.mark.parametrize("shape,kernel,causal,head_dim", [
    ((16, 16), (5, 5), (False, True), 64),     # backward on the original tensors, dQ + combined dK/dV role
    ((16, 32), (7, 9), (True, False), 128),    # the same with the paired dK/dV role
    ((20, 24), (5, 7), (False, False), 64),    # permutes + backward kernels + unpermutes
])
def test_training_step_replays_from_a_graph(shape, kernel, causal, head_dim):
    # forward and backward captured together; the gradients of every replay (new inputs copied
    # into the captured tensors) equal those of the eager step bit for bit
    gen = torch.Generator().manual_seed(1)
    mk = lambda: torch.randn((1, *shape, 2, head_dim), generator=gen).to(torch.bfloat16).cuda()
    q, k, v = (mk().requires_grad_(True) for _ in range(3))
    d_out = mk()

    def step(a, b, c):
        natten_amd.na2d(a, b, c, kernel, is_causal=causal).backward(d_out)

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for _ in range(2):  # warm-up outside the capture
            step(q, k, v)
    torch.cuda.current_stream().wait_stream(side)
    for t in (q, k, v):
        t.grad = None  # the captured backward allocates the gradients from the graph's pool
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(q, k, v)
    for i in range(3):
        with torch.no_grad():
            for t in (q, k, v, d_out):
                t.copy_(mk())
        graph.replay()
        torch.cuda.synchronize()
        eager = [t.detach().clone().requires_grad_(True) for t in (q, k, v)]
        step(*eager)   # eager work between the replays
        torch.cuda.synchronize()
        for name, a, b in zip("qkv", (q, k, v), eager):
            assert torch.equal(a.grad, b.grad), f"replay {i}: d{name} differs from the eager step"


def test_varlen_training_step_replays_from_a_graph():
    # sequence-packed attention: the backward builds its padded packing with device index
    # arithmetic (cumsum, searchsorted, index_copy_), all of which must replay correctly
    gen = torch.Generator().manual_seed(2)
    mk = lambda: torch.randn((1, 300, 2, 64), generator=gen).to(torch.bfloat16).cuda()
    q, k, v = (mk().requires_grad_(True) for _ in range(3))
    d_out = mk()
    cu = torch.tensor([0, 40, 170, 300], dtype=torch.int32, device="cuda")

    def step(a, b, c):
        natten_amd.attention(a, b, c, is_causal=True, cumulative_seqlen_Q=cu, cumulative_seqlen_KV=cu,
                             max_seqlen_Q=130, max_seqlen_KV=130).backward(d_out)

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for _ in range(2):
            step(q, k, v)
    torch.cuda.current_stream().wait_stream(side)
    for t in (q, k, v):
        t.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(q, k, v)
    for i in range(3):
        with torch.no_grad():
            for t in (q, k, v, d_out):
                t.copy_(mk())
        graph.replay()
        torch.cuda.synchronize()
        eager = [t.detach().clone().requires_grad_(True) for t in (q, k, v)]
        step(*eager)
        torch.cuda.synchronize()
        for name, a, b in zip("qkv", (q, k, v), eager):
            assert torch.equal(a.grad, b.grad), f"replay {i}: d{name} differs from the eager step"
