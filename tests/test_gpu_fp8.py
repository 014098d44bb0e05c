"""GPU parity for quantised 8-bit float operands (e4m3fn / e5m2 with per-head scales).

The attention results are compared with the float64 oracle evaluated on the DEQUANTISED inputs.
Two routes, two stated tolerances:
  * 8-bit matrix instruction (default when head dim and tiles allow), P rounded to e4m3 as the
    reference does.  Each probability then carries a relative error of up to 2^-4 (half a unit
    of its 3-bit mantissa), so |out - ref| <= 2^-4 * max|V| holds for every element whatever the
    window (checked as the absolute tolerance), and over a whole tensor the errors average out:
    rms(out - ref) <= 3e-2 * rms(ref) (checked; observed 1.9e-2 to 2.5e-2).  LSE is computed
    from unrounded probabilities: atol = rtol = 1e-2 as for 16-bit operands (observed 2e-5).
    The reference tests the same arithmetic with atol 0.5 (tests/test_blackwell_fna.py:107).
  * fp8_matmul=False: operands widened exactly to bf16 by the token permute (bit-exact, every
    8-bit float value is a bf16 value) and multiplied in bf16: atol = rtol = 1e-2, as for bf16."""

import numpy as np
import pytest
import torch

import natten_amd
from natten_amd import _lib
from oracle import c_oracle
from oracle import na_oracle as O
from tests.gpu_utils import assert_close, stratified_tokens, to_np

pytestmark = pytest.mark.gpu

E4M3_MAX = 448.0
E5M2_MAX = 57344.0


def check_out(name, fp8_matmul, got, ref, v_dequantised):
    """Output tolerance of the two routes (see the module docstring)."""
    if fp8_matmul is False:
        assert_close(name, got, ref)
        return
    bound = 2.0**-4 * float(v_dequantised.abs().max())
    assert_close(name, got, ref, atol=bound, rtol=0.0)
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    rms_err, rms_ref = np.sqrt(((got - ref) ** 2).mean()), np.sqrt((ref**2).mean())
    assert rms_err <= 3e-2 * rms_ref, f"{name}: rms error {rms_err:.4e} above 3e-2 of rms(ref) {rms_ref:.4e}"



def quantise_per_head(x, dtype):
    """Per-head absmax scaling into the 8-bit range: returns (x8, scale[H]) with x ~ x8 * scale."""
    fmax = E4M3_MAX if dtype == torch.float8_e4m3fn else E5M2_MAX
    red = tuple(i for i in range(x.dim()) if i != x.dim() - 2)
    scale = x.abs().amax(dim=red).float() / fmax
    x8 = (x / scale.view(*([1] * (x.dim() - 2)), -1, 1)).to(dtype)
    return x8, scale


def dequantise(x8, scale):
    return x8.float() * scale.view(*([1] * (x8.dim() - 2)), -1, 1)


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_widen_all_byte_values_bit_exact(dtype):
    # every byte value, laid out as [B=1, S=32, H=1, D=8]
    raw = torch.arange(256, dtype=torch.uint8, device="cuda").reshape(1, 32, 1, 8)
    x = raw.view(dtype)
    got = _lib.token_permute(x, (1,), (1,), True, widen=True)
    ref = x.to(torch.bfloat16)
    assert got.dtype == torch.bfloat16 and got.shape == ref.shape
    nan = torch.isnan(ref)
    assert torch.equal(torch.isnan(got), nan)
    assert torch.equal(got.view(torch.int16)[~nan], ref.view(torch.int16)[~nan])


@pytest.mark.parametrize(
    "shape,tile,dil",
    [((37,), (8,), (1,)), ((19, 23), (4, 8), (2, 3)), ((5, 9, 11), (2, 4, 4), (1, 2, 2)), ((16, 16), (8, 8), (1, 1))],
)
def test_widen_permute_matches_oracle(shape, tile, dil):
    gen = torch.Generator().manual_seed(3)
    x = torch.randn((2, *shape, 3, 16), generator=gen).to(torch.float8_e4m3fn).cuda()
    got = _lib.token_permute(x, tile, dil, True, widen=True)
    ref, _, _ = O.token_permute(to_np(x), tile, dil, flip=True)
    assert got.dtype == torch.bfloat16
    assert np.array_equal(to_np(got), ref)
    # and the plain permute of the same tensor carries the bytes verbatim
    raw = _lib.token_permute(x, tile, dil, True)
    assert raw.dtype == x.dtype
    assert np.array_equal(to_np(raw), ref)


def _sampled(qd, kd, vd, out, lse, kernel, stride, dilation, causal, n_samples, seed, fp8_matmul=False):
    B = qd.shape[0]
    n = qd.dim() - 3
    N = int(np.prod(qd.shape[1 : 1 + n]))
    H, D = qd.shape[-2], qd.shape[-1]
    rng = np.random.default_rng(seed)
    tok = stratified_tokens(tuple(qd.shape[1 : 1 + n]), kernel, stride, dilation, causal, n_samples, rng)
    bat = rng.integers(0, B, size=len(tok))
    ref_o, ref_l, _ = c_oracle.na_rows(to_np(qd), to_np(kd), to_np(vd), kernel, stride, dilation, causal, None, bat,
                                       tok, threads=16)
    ti, bi = torch.as_tensor(tok), torch.as_tensor(bat)
    check_out("sampled out", fp8_matmul, to_np(out.reshape(B, N, H, D)[bi, ti]), ref_o, vd)
    assert_close("sampled lse", to_np(lse.reshape(B, N, H)[bi, ti]), ref_l)


@pytest.mark.parametrize("fp8_matmul", [True, False])
def test_config5_e4m3_full_size_sampled(fp8_matmul):
    # na3d e4m3, B=1, heads 16, 16x64x64, D=128, kernel (8,16,16), stride (4,8,8), dilation (1,2,2)
    gen = torch.Generator().manual_seed(0)
    shape, H, D = (16, 64, 64), 16, 128
    q, k, v = (torch.randn((1, *shape, H, D), generator=gen).cuda() for _ in range(3))
    (q8, sq), (k8, sk), (v8, sv) = (quantise_per_head(t, torch.float8_e4m3fn) for t in (q, k, v))
    args = ((8, 16, 16), (4, 8, 8), (1, 2, 2))
    with torch.no_grad():
        out, lse = natten_amd.na3d(q8, k8, v8, *args, return_lse=True, q_scale=sq, k_scale=sk, v_scale=sv,
                                   out_dtype=torch.bfloat16, fp8_matmul=fp8_matmul)
    assert out.dtype == torch.bfloat16 and lse.dtype == torch.float32
    qd, kd, vd = dequantise(q8, sq), dequantise(k8, sk), dequantise(v8, sv)
    _sampled(qd, kd, vd, out, lse, *args, (False, False, False), n_samples=2000, seed=5, fp8_matmul=fp8_matmul)
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    # doubling v_scale doubles the output bit-exactly and leaves LSE alone
    with torch.no_grad():
        out2, lse2 = natten_amd.na3d(q8, k8, v8, *args, return_lse=True, q_scale=sq, k_scale=sk, v_scale=sv * 2,
                                     out_dtype=torch.bfloat16, fp8_matmul=fp8_matmul)
    assert torch.equal(out2, out * 2) and torch.equal(lse2, lse)


@pytest.mark.parametrize("fp8_matmul", [True, False])
@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("causal", [False, True])
def test_small_fp8_problems_match_oracle(dtype, causal, fp8_matmul):
    gen = torch.Generator().manual_seed(11)
    B, shape, H, Hkv, D = 2, (14, 20), 4, 2, 48
    q = torch.randn((B, *shape, H, D), generator=gen).cuda()
    k = torch.randn((B, *shape, Hkv, D), generator=gen).cuda()
    v = torch.randn((B, *shape, Hkv, D), generator=gen).cuda()
    (q8, sq), (k8, sk), (v8, sv) = (quantise_per_head(t, dtype) for t in (q, k, v))
    kernel, stride, dil, cz = (5, 6), (2, 3), (2, 1), (causal, False)
    with torch.no_grad():
        out, lse = natten_amd.na2d(q8, k8, v8, kernel, stride, dil, cz, return_lse=True, q_scale=sq, k_scale=sk,
                                   v_scale=sv, out_dtype=torch.bfloat16, fp8_matmul=fp8_matmul)
    qd, kd, vd = dequantise(q8, sq), dequantise(k8, sk), dequantise(v8, sv)
    ref_o, ref_l = c_oracle.na_forward(to_np(qd), to_np(kd), to_np(vd), kernel, stride, dil, cz, None)
    check_out("out", fp8_matmul, to_np(out), ref_o, vd)
    assert_close("lse", to_np(lse), ref_l)


def test_fp8_default_output_dtype_and_unit_scales():
    # without scales and out_dtype the call behaves like the reference: 8-bit result
    gen = torch.Generator().manual_seed(2)
    q, k, v = ((torch.randn((1, 40, 2, 32), generator=gen) * 0.5).to(torch.float8_e4m3fn).cuda() for _ in range(3))
    with torch.no_grad():
        out, lse = natten_amd.na1d(q, k, v, 9, return_lse=True)
    assert out.dtype == torch.float8_e4m3fn
    ref_o, ref_l = c_oracle.na_forward(to_np(q), to_np(k), to_np(v), (9,), (1,), (1,), (False,), None)
    # the result is rounded to e4m3 (3 mantissa bits: relative step 2^-3, half of it as error)
    assert_close("out", to_np(out), ref_o, atol=2e-2, rtol=2.0**-4)
    assert_close("lse", to_np(lse), ref_l)


def test_fp8_dense_attention_and_additional_kv():
    gen = torch.Generator().manual_seed(4)
    B, L, H, D = 1, 70, 2, 64
    q, k, v = (torch.randn((B, L, H, D), generator=gen).cuda() for _ in range(3))
    ak, av = (torch.randn((B, 13, H, D), generator=gen).cuda() for _ in range(2))
    (q8, sq), (k8, sk), (v8, sv) = (quantise_per_head(t, torch.float8_e4m3fn) for t in (q, k, v))
    # the additional tensors share the scales of key / value
    ak8 = (ak / sk.view(1, 1, -1, 1)).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    av8 = (av / sv.view(1, 1, -1, 1)).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    qd, kd, vd = dequantise(q8, sq), dequantise(k8, sk), dequantise(v8, sv)
    akd, avd = dequantise(ak8, sk), dequantise(av8, sv)
    with torch.no_grad():
        out, lse = natten_amd.attention(q8, k8, v8, return_lse=True, q_scale=sq, k_scale=sk, v_scale=sv,
                                        out_dtype=torch.bfloat16)
    ref_o, ref_l = O.attention_forward(to_np(qd), to_np(kd), to_np(vd))
    assert_close("dense out", to_np(out), ref_o)
    assert_close("dense lse", to_np(lse), ref_l)
    ref_o, ref_l = O.na_forward(to_np(qd), to_np(kd), to_np(vd), (7,), additional_keys=to_np(akd),
                                additional_values=to_np(avd))
    for fp8_matmul in (False, None):
        with torch.no_grad():
            out, lse = natten_amd.na1d(q8, k8, v8, 7, additional_keys=ak8, additional_values=av8, return_lse=True,
                                       q_scale=sq, k_scale=sk, v_scale=sv, out_dtype=torch.bfloat16,
                                       fp8_matmul=fp8_matmul)
        check_out("na + additional out", fp8_matmul, to_np(out), ref_o, torch.cat([vd, avd], dim=1))
        assert_close("na + additional lse", to_np(lse), ref_l)


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("D", [64, 128])
def test_fp8_matmul_fused_equals_permuted(dtype, D):
    # the 8-bit kernel on the original tensors and on token-permuted bytes: bit-identical
    from natten_amd.fna import amd_fna_generic

    gen = torch.Generator().manual_seed(9)
    shape, H, Hkv = (4, 16, 32), 4, 2
    q = torch.randn((2, *shape, H, D), generator=gen).cuda()
    k = torch.randn((2, *shape, Hkv, D), generator=gen).cuda()
    v = torch.randn((2, *shape, Hkv, D), generator=gen).cuda()
    (q8, sq), (k8, sk), (v8, sv) = (quantise_per_head(t, dtype) for t in (q, k, v))
    args = ((3, 7, 9), (1, 2, 3), (1, 2, 1), (True, False, False))
    kw = dict(q_tile_shape=(2, 8, 8), kv_tile_shape=(2, 4, 8), return_lse=True, q_scale=sq, k_scale=sk, v_scale=sv,
              out_dtype=torch.bfloat16, fp8_matmul=True)
    with torch.no_grad():
        out_f, lse_f = amd_fna_generic(q8, k8, v8, *args, fused=True, anchored_tiles=False, **kw)
        out_p, lse_p = amd_fna_generic(q8, k8, v8, *args, fused=False, **kw)
        out_a, lse_a = amd_fna_generic(q8, k8, v8, *args, fused=True, anchored_tiles=True, **kw)
        # work-queue launch of the 8-bit kernel: the same bits as a workgroup per Q tile, on both layouts
        out_aq, lse_aq = amd_fna_generic(q8, k8, v8, *args, fused=True, run_persistent_kernel=True, **kw)
        out_pq, lse_pq = amd_fna_generic(q8, k8, v8, *args, fused=False, run_persistent_kernel=True, **kw)
    assert torch.equal(out_f, out_p) and torch.equal(lse_f, lse_p)
    assert torch.equal(out_aq, out_a) and torch.equal(lse_aq, lse_a)
    assert torch.equal(out_pq, out_p) and torch.equal(lse_pq, lse_p)
    qd, kd, vd = dequantise(q8, sq), dequantise(k8, sk), dequantise(v8, sv)
    ref_o, ref_l = c_oracle.na_forward(to_np(qd), to_np(kd), to_np(vd), *args, None)
    check_out("out", True, to_np(out_f), ref_o, vd)
    assert_close("lse", to_np(lse_f), ref_l)
    # KV tiles laid out from the window's first key (the default on the original tensors)
    check_out("out, anchored tiles", True, to_np(out_a), ref_o, vd)
    assert_close("lse, anchored tiles", to_np(lse_a), ref_l)


@pytest.mark.parametrize("shape,kernel,stride,dilation,causal", [
    ((5, 18, 30), (3, 7, 9), (1, 2, 3), (1, 2, 1), (True, False, False)),   # extents no tile shape divides
    ((37, 50), (9, 12), (2, 4), (1, 3), (False, True)),                      # uneven dilation groups
    ((333,), (65,), (8,), (2,), (False,)),
])
def test_fp8_odd_extents_work_queue_equals_per_tile(shape, kernel, stride, dilation, causal):
    # whatever route the driver picks for extents the tiles do not divide, the 8-bit kernel's
    # work-queue launch gives the bits of the one-workgroup-per-tile launch, and both match the oracle
    from natten_amd.fna import amd_fna_generic

    gen = torch.Generator().manual_seed(21)
    H, Hkv, D = 4, 2, 128
    q = torch.randn((2, *shape, H, D), generator=gen).cuda()
    k = torch.randn((2, *shape, Hkv, D), generator=gen).cuda()
    v = torch.randn((2, *shape, Hkv, D), generator=gen).cuda()
    (q8, sq), (k8, sk), (v8, sv) = (quantise_per_head(t, torch.float8_e4m3fn) for t in (q, k, v))
    kw = dict(return_lse=True, q_scale=sq, k_scale=sk, v_scale=sv, out_dtype=torch.bfloat16, fp8_matmul=True)
    with torch.no_grad():
        out_t, lse_t = amd_fna_generic(q8, k8, v8, kernel, stride, dilation, causal, run_persistent_kernel=False, **kw)
        for _ in range(2):
            out_q, lse_q = amd_fna_generic(q8, k8, v8, kernel, stride, dilation, causal, run_persistent_kernel=True, **kw)
            assert torch.equal(out_q, out_t) and torch.equal(lse_q, lse_t)
    qd, kd, vd = dequantise(q8, sq), dequantise(k8, sk), dequantise(v8, sv)
    ref_o, ref_l = c_oracle.na_forward(to_np(qd), to_np(kd), to_np(vd), kernel, stride, dilation, causal, None)
    check_out("out", True, to_np(out_q), ref_o, vd)
    assert_close("lse", to_np(lse_q), ref_l)
    # where every dilation group is at least a KV tile wide the 8-bit kernel takes these extents in
    # one launch on the original tensors (edge tiles moved back); the permuted route meets the same bar
    from natten_amd import _lib
    from natten_amd.tile_config import check_fna_forward_config

    qt, kt = check_fna_forward_config(q8, kernel, stride, dilation, causal, None, None)
    if all(X // d >= t for X, d, t in zip(shape, dilation, kt)):
        assert _lib.fused_layout_supported(shape, dilation, kt, row_bytes=Hkv * D * 2, q_tile_shape=qt, dtype=q8.dtype)
        with torch.no_grad():
            out_f, lse_f = amd_fna_generic(q8, k8, v8, kernel, stride, dilation, causal, fused=True, **kw)
            out_p, lse_p = amd_fna_generic(q8, k8, v8, kernel, stride, dilation, causal, fused=False, **kw)
        assert torch.equal(out_f, out_q) and torch.equal(lse_f, lse_q)
        check_out("out (permuted route)", True, to_np(out_p), ref_o, vd)
        assert_close("lse (permuted route)", to_np(lse_p), ref_l)


def test_fp8_matmul_rejects_unsupported_shapes():
    from natten_amd.fna import amd_fna_generic

    q, k, v = (torch.zeros((1, 64, 2, 32), dtype=torch.float8_e4m3fn, device="cuda") for _ in range(3))
    with pytest.raises(ValueError):
        amd_fna_generic(q, k, v, (9,), fp8_matmul=True)  # head_dim 32 has no 8-bit instance
