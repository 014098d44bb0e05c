"""GPU parity: dense attention, attention merge, additional keys/values and the self-attention
fast path, through the public API (C ABI underneath), against the CPU oracle.
Tolerance atol = rtol = 1e-2 (fp16 / bf16 operands, float64 oracle on the same rounded inputs)."""

import numpy as np
import pytest
import torch

import natten_amd
from oracle import na_oracle as O
from tests.gpu_utils import assert_close, make_qkv, to_np

pytestmark = pytest.mark.gpu


def _rand(shape, dtype, seed, std=1.0):
    gen = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=gen) * std).to(dtype).cuda()


ATTN_CASES = [
    # B, Sq, Skv, H, Hkv, D, causal
    (2, 128, 128, 4, 4, 64, False),
    (1, 125, 300, 2, 1, 128, False),
    (1, 300, 125, 2, 2, 32, False),
    (2, 77, 77, 3, 3, 64, True),
    (1, 513, 513, 2, 1, 128, True),
    (1, 200, 64, 2, 2, 64, True),   # causal with fewer keys than queries (top-left aligned)
    (1, 1, 1, 1, 1, 32, False),
    (1, 5, 1, 2, 2, 64, True),
    (1, 130, 9, 4, 2, 48, False),   # head_dim that is padded to 64 internally
    (1, 64, 1000, 1, 1, 120, False),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_attention_matches_oracle(dtype):
    for i, (B, Sq, Skv, H, Hkv, D, causal) in enumerate(ATTN_CASES):
        q = _rand((B, Sq, H, D), dtype, 3 * i)
        k = _rand((B, Skv, Hkv, D), dtype, 3 * i + 1)
        v = _rand((B, Skv, Hkv, D), dtype, 3 * i + 2)
        with torch.no_grad():
            out, lse = natten_amd.attention(q, k, v, is_causal=causal, return_lse=True)
            only = natten_amd.attention(q, k, v, is_causal=causal)
        torch.cuda.synchronize()
        assert isinstance(only, torch.Tensor) and torch.equal(only, out)
        ref_o, ref_l = O.attention_forward(to_np(q), to_np(k), to_np(v), is_causal=causal)
        tag = f"attention {(B, Sq, Skv, H, Hkv, D, causal)} {dtype}"
        assert_close("out " + tag, to_np(out), ref_o)
        assert_close("lse " + tag, to_np(lse), ref_l)


def test_attention_custom_scale():
    q, k, v = (_rand((1, 96, 2, 64), torch.bfloat16, s) for s in (1, 2, 3))
    with torch.no_grad():
        out, lse = natten_amd.attention(q, k, v, scale=0.05, return_lse=True)
    ref_o, ref_l = O.attention_forward(to_np(q), to_np(k), to_np(v), scale=0.05)
    assert_close("out", to_np(out), ref_o)
    assert_close("lse", to_np(lse), ref_l)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_merge_attentions_matches_oracle(dtype):
    gen = torch.Generator().manual_seed(5)
    outs = [torch.randn((2, 50, 3, 64), generator=gen).to(dtype).cuda() for _ in range(3)]
    lses = [(torch.randn((2, 50, 3), generator=gen) * 3).cuda() for _ in range(3)]
    for n in (2, 3):
        with torch.no_grad():
            o, l = natten_amd.merge_attentions(outs[:n], lses[:n])
        ref_o, ref_l = O.merge_attentions([to_np(x) for x in outs[:n]], [to_np(x) for x in lses[:n]])
        assert o.dtype == dtype and l.dtype == torch.float32
        assert_close(f"merge out n={n} {dtype}", to_np(o), ref_o)
        assert_close(f"merge lse n={n} {dtype}", to_np(l), ref_l, atol=1e-5, rtol=1e-5)


def test_merge_of_split_attention_equals_whole():
    # tests/test_attn_merge.py:51-113 pattern of the reference: split the keys, attend, merge
    q = _rand((1, 200, 2, 64), torch.bfloat16, 1)
    k = _rand((1, 333, 2, 64), torch.bfloat16, 2)
    v = _rand((1, 333, 2, 64), torch.bfloat16, 3)
    with torch.no_grad():
        parts = [natten_amd.attention(q, k[:, a:b], v[:, a:b], return_lse=True) for a, b in ((0, 100), (100, 333))]
        o, l = natten_amd.merge_attentions([p[0] for p in parts], [p[1] for p in parts])
    ref_o, ref_l = O.attention_forward(to_np(q), to_np(k), to_np(v))
    assert_close("out", to_np(o), ref_o, atol=2e-2, rtol=2e-2)  # two roundings of partial outputs to bf16
    assert_close("lse", to_np(l), ref_l)


def test_merge_argument_errors():
    o = torch.zeros(1, 4, 2, 8).cuda()
    l = torch.zeros(1, 4, 2).cuda()
    with pytest.raises(ValueError):
        natten_amd.merge_attentions([o], [l])
    with pytest.raises(ValueError):
        natten_amd.merge_attentions([o, o], [l])
    with pytest.raises(ValueError):
        natten_amd.merge_attentions([o, o[:, :2]], [l, l])
    with pytest.raises(ValueError):
        natten_amd.merge_attentions([o, o], [l, l[..., None]])


@pytest.mark.parametrize("na_dim", [1, 2, 3])
def test_additional_keys_values(na_dim):
    shape = {1: (100,), 2: (12, 20), 3: (5, 8, 12)}[na_dim]
    k = {1: (9,), 2: (5, 7), 3: (3, 3, 5)}[na_dim]
    q, kk, v = make_qkv(2, shape, 4, 2, 64, torch.bfloat16, seed=7)
    ak = _rand((2, 37, 2, 64), torch.bfloat16, 8)
    av = _rand((2, 37, 2, 64), torch.bfloat16, 9)
    fn = {1: natten_amd.na1d, 2: natten_amd.na2d, 3: natten_amd.na3d}[na_dim]
    with torch.no_grad():
        out, lse = fn(q, kk, v, k, additional_keys=ak, additional_values=av, return_lse=True)
    ref_o, ref_l = O.na_forward(to_np(q), to_np(kk), to_np(v), k, additional_keys=to_np(ak), additional_values=to_np(av))
    assert_close("out", to_np(out), ref_o, atol=2e-2, rtol=2e-2)  # partial outputs are rounded before the merge
    assert_close("lse", to_np(lse), ref_l)
    with pytest.raises(ValueError):
        fn(q, kk, v, k, additional_keys=ak)


def test_full_window_takes_the_attention_path():
    # kernel_size == input size, non-causal: plain attention over the flattened tokens
    q, kk, v = make_qkv(1, (8, 12), 2, 2, 64, torch.float16, seed=3)
    with torch.no_grad():
        out, lse = natten_amd.na2d(q, kk, v, (8, 12), return_lse=True)
    ref_o, ref_l = O.na_forward(to_np(q), to_np(kk), to_np(v), (8, 12))
    assert_close("out", to_np(out), ref_o)
    assert_close("lse", to_np(lse), ref_l)
    # 1-D full window, causal: causal attention
    q, kk, v = make_qkv(1, (150,), 2, 1, 32, torch.bfloat16, seed=4)
    with torch.no_grad():
        out, lse = natten_amd.na1d(q, kk, v, 150, is_causal=True, return_lse=True)
    ref_o, ref_l = O.na_forward(to_np(q), to_np(kk), to_np(v), (150,), is_causal=(True,))
    assert_close("out", to_np(out), ref_o)
    assert_close("lse", to_np(lse), ref_l)
    # with additional context the extra tokens join the key sequence
    ak, av = _rand((1, 20, 2, 64), torch.float16, 5), _rand((1, 20, 2, 64), torch.float16, 6)
    q, kk, v = make_qkv(1, (8, 12), 2, 2, 64, torch.float16, seed=3)
    with torch.no_grad():
        out, lse = natten_amd.na2d(q, kk, v, (8, 12), additional_keys=ak, additional_values=av, return_lse=True)
    ref_o, ref_l = O.na_forward(to_np(q), to_np(kk), to_np(v), (8, 12), additional_keys=to_np(ak), additional_values=to_np(av))
    assert_close("out", to_np(out), ref_o)
    assert_close("lse", to_np(lse), ref_l)


def test_attention_errors():
    q = torch.zeros(1, 16, 2, 64, dtype=torch.bfloat16).cuda()
    with pytest.raises(ValueError):
        natten_amd.attention(q, q[:, :, :1], q)
    with pytest.raises(ValueError):
        natten_amd.attention(q, q[:, :8], q)
    with pytest.raises(ValueError):  # cumulative lengths without their partner and the maxima
        natten_amd.attention(q, q, q, cumulative_seqlen_Q=torch.zeros(2, dtype=torch.int32))
    with pytest.raises(NotImplementedError):
        natten_amd.attention(q.float(), q.float(), q.float())


def test_mfma_probe_reports_plausible_rates():
    # diagnostic entry point: constant operands run at a higher clock than random ones, and
    # neither exceeds the data-sheet peak
    from natten_amd import _lib

    rnd, rnd_ghz = _lib.mfma_probe(random_operands=True, iters=2000)
    const, const_ghz = _lib.mfma_probe(random_operands=False, iters=2000)
    assert 100.0 < rnd < 2600.0 and 100.0 < const < 2600.0
    assert 0.3 < rnd_ghz < 2.6 and 0.3 < const_ghz < 2.6


def test_neighborhood_attention_layer_matches_its_parts():
    # the layer = qkv projection, na2d, output projection (reference src/natten/modules.py:83-123)
    import natten_amd

    torch.manual_seed(0)
    layer = natten_amd.NeighborhoodAttention2D(embed_dim=128, num_heads=4, kernel_size=(5, 7), stride=(1, 2),
                                               is_causal=(False, True)).cuda().to(torch.bfloat16)
    x = torch.randn(2, 16, 24, 128, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        y = layer(x)
        qkv = layer.qkv(x).reshape(2, 16, 24, 3, 4, 32)
        ref = layer.proj(natten_amd.na2d(qkv[:, :, :, 0], qkv[:, :, :, 1], qkv[:, :, :, 2], (5, 7), (1, 2), 1,
                                         (False, True)).reshape(2, 16, 24, 128))
    assert y.shape == x.shape and torch.equal(y, ref)
    with pytest.raises(ValueError):
        layer(x[0])
    assert set(layer.state_dict()) == {"qkv.weight", "qkv.bias", "proj.weight", "proj.bias"}
