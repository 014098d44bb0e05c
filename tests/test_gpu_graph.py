"""The forward under HIP graph capture: the entry points allocate nothing and launch on the
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
