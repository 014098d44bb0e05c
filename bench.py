"""Benchmark of the MI355X neighborhood attention forward path.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4|c3|c2|c2d]

One step = one na3d/na2d forward through the public API on inputs already resident in HBM:
a single launch that gathers its tiles from the original tensors when the problem allows it
(all benchmark workloads do), else token permute of Q/K/V, kernel, unpermute of O and LSE.  Prints ONE JSON line: whole-path throughput in effective
NA TFLOP/s (4 * B * H * D * sum_q |window(q)| per step), the fused kernel's roofline figures from
HIP-event timing of kernel-only launches, and a CPU baseline (the C oracle on a bounded sample
of the same workload's queries, timed on this box's host cores).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X dense MFMA peak of the instruction the path multiplies with
PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "e4m3": 5000.0}

WORKLOADS = {
    # name: (B, H, layout, D, kernel, stride, dilation, causal, dtype, std)
    "c4": (1, 24, (30, 48, 80), 128, (18, 24, 24), (1, 8, 8), (1, 1, 1), (True, False, False), "bf16", 1.0),
    "c3": (1, 16, (128, 128), 128, (32, 32), (16, 16), (1, 1), (False, False), "fp16", 0.5),
    "c2": (2, 8, (64, 64), 64, (13, 13), (1, 1), (1, 1), (False, False), "bf16", 1.0),
    "c2d": (2, 8, (64, 64), 64, (13, 13), (1, 1), (2, 2), (False, False), "bf16", 1.0),
    # e4m3 operands with per-head absmax scales, bf16 output; multiplied by the 8-bit matrix instruction
    "c5": (1, 16, (16, 64, 64), 128, (8, 16, 16), (4, 8, 8), (1, 2, 2), (False, False, False), "e4m3", 1.0),
}
# HBM-side traffic of one fused-kernel launch, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# and calibrated on the permute kernel (a copy of known size); the summary of that run is kept with the profiles.
# Keyed by (workload, q_tile_shape, kv_tile_shape); other combinations report null.
MEASURED_TRAFFIC_BYTES = {
    ("c4", (2, 8, 8), (1, 8, 8)): 2.82e10,
}
# The same for the two backward launches together (dQ role 20.3 GB read + 0.7 GB written, paired
# dK / dV role 63.7 GB + 1.9 GB), keyed by (workload, backward q tile, backward kv tile).
MEASURED_BACKWARD_TRAFFIC_BYTES = {
    ("c4", (2, 8, 8), (2, 8, 8)): 8.66e10,
}

WORKLOAD_NAMES = {
    "c4": "na3d bf16 B=1 H=24 30x48x80 D=128 k=(18,24,24) s=(1,8,8) causal=(T,F,F) +LSE",
    "c3": "na2d fp16 B=1 H=16 128x128 D=128 k=(32,32) s=(16,16)",
    "c2": "na2d bf16 B=2 H=8 64x64 D=64 k=(13,13)",
    "c2d": "na2d bf16 B=2 H=8 64x64 D=64 k=(13,13) d=(2,2)",
    "c5": "na3d e4m3 (per-head scales, bf16 out) B=1 H=16 16x64x64 D=128 k=(8,16,16) s=(4,8,8) d=(1,2,2)",
}


def count_attended(layout, k, s, d, c):
    # closed-form sum over queries of window sizes (product of per-dimension sums)
    def win(i, kk, ss, L, causal):
        wl, wr = kk // 2, kk // 2 + (kk % 2 - 1)
        if causal:
            leader = min((i // ss) * ss + ss - 1, L - 1)
            return min(i + 1, L) - max(leader - wl - wr, 0)
        return kk

    total = 1
    for X, kk, ss, dd, cc in zip(layout, k, s, d, c):
        acc = 0
        for g in range(dd):
            L = X // dd + 1 - ((g + (dd - X % dd)) // dd)
            acc += sum(win(i, kk, ss, L, cc) for i in range(L))
        total *= acc
    return total


def cpu_baseline(q, k, v, kernel, stride, dilation, causal, out_gpu, lse_gpu, seconds_target=15.0, tol=1e-2):
    """C oracle on a bounded sample of this workload's queries, all heads, host cores."""
    import numpy as np

    from oracle import c_oracle

    B = q.shape[0]
    n = q.dim() - 3
    N = 1
    for x in q.shape[1 : 1 + n]:
        N *= int(x)
    H, D = q.shape[-2], q.shape[-1]
    threads = min(16, os.cpu_count() or 1)
    qn, kn, vn = (t.float().cpu().numpy() for t in (q, k, v))
    rng = np.random.default_rng(0)
    # calibrate on a few queries, then size the sample for ~seconds_target of wall time
    probe = rng.integers(0, N, size=threads)
    t0 = time.perf_counter()
    c_oracle.na_rows(qn, kn, vn, kernel, stride, dilation, causal, None, np.zeros_like(probe), probe, threads)
    dt = max(time.perf_counter() - t0, 1e-4)
    nq = int(max(threads, min(N * B, threads * seconds_target / dt)))
    tok = rng.integers(0, N, size=nq)
    bat = rng.integers(0, B, size=nq)
    t0 = time.perf_counter()
    ref_o, ref_l, visited = c_oracle.na_rows(qn, kn, vn, kernel, stride, dilation, causal, None, bat, tok, threads)
    dt = time.perf_counter() - t0
    flops = 4.0 * D * visited
    got_o = out_gpu.reshape(B, N, H, D)[torch_idx(bat), torch_idx(tok)].float().cpu().numpy()
    got_l = lse_gpu.reshape(B, N, H)[torch_idx(bat), torch_idx(tok)].float().cpu().numpy()
    err_o = float(np.abs(got_o - ref_o).max())
    err_l = float(np.abs(got_l - ref_l).max())
    ok = bool(((np.abs(got_o - ref_o) <= tol + tol * np.abs(ref_o)).all())
              and ((np.abs(got_l - ref_l) <= 1e-2 + 1e-2 * np.abs(ref_l)).all()))
    return {
        "value": flops / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"C oracle (float64), {nq} random queries x {H} heads of this workload, {dt:.1f} s wall",
        "parity_on_sample": {"ok": ok, "max_abs_err_out": err_o, "max_abs_err_lse": err_l, "atol_rtol": tol},
    }


def torch_idx(a):
    import torch

    return torch.as_tensor(a, dtype=torch.long)


def bench_backward(args, q, k, v, kernel, stride, dilation, causal, dt_name):
    """Secondary measurement: one step = forward + backward through the public API; the backward
    kernels (dQ role + dK/dV role of fna_bwd_kernel) are timed on their own with HIP events.
    Work is counted as 2.5 x the forward's algorithmic FLOP (five matrix products against two)."""
    import torch

    import natten_amd
    from natten_amd import _lib
    from natten_amd.tile_config import check_fna_backward_config
    from natten_amd.token_permute import token_permute_operation

    n = q.dim() - 3
    B, H, D = q.shape[0], q.shape[-2], q.shape[-1]
    layout = tuple(q.shape[1 : 1 + n])
    na = {1: natten_amd.na1d, 2: natten_amd.na2d, 3: natten_amd.na3d}[n]
    q_tile = tuple(int(x) for x in args.q_tile.split(",")) if args.q_tile else None
    kv_tile = tuple(int(x) for x in args.kv_tile.split(",")) if args.kv_tile else None
    q_tile, kv_tile = check_fna_backward_config(q, kernel, stride, dilation, causal, q_tile, kv_tile)
    gen = torch.Generator().manual_seed(1)
    d_out = torch.randn(q.shape, generator=gen).to(q.dtype).to(q.device)
    q, k, v = (t.clone().requires_grad_(True) for t in (q, k, v))

    def step():
        q.grad = k.grad = v.grad = None
        out = na(q, k, v, kernel, stride, dilation, causal, backward_q_tile_shape=q_tile,
                 backward_kv_tile_shape=kv_tile)
        out.backward(d_out)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    with torch.no_grad():
        out, lse = na(q, k, v, kernel, stride, dilation, causal, return_lse=True)
        delta = _lib.compute_delta(out, d_out)

        def perm(x, t):
            return token_permute_operation(x.contiguous(), t, dilation, flip_tiled_dims=True)

        qp, qkv_shape, q_shape = perm(q, q_tile)
        dop = perm(d_out, q_tile)[0]
        lp = perm(lse.unsqueeze(-1), q_tile)[0].squeeze(-1).contiguous()
        dp = perm(delta.unsqueeze(-1), q_tile)[0].squeeze(-1).contiguous()
        kp, _, kv_shape = perm(k, kv_tile)
        vp = perm(v, kv_tile)[0]

        fused = _lib.backward_fused_layout_supported(layout, dilation, q_tile, kv_tile)
        qd, kd, vd = q.detach(), k.detach(), v.detach()

        def kern_permuted():
            return _lib.fna_backward(qp, kp, vp, dop, lp, dp, kernel, stride, dilation, causal, D**-0.5, q_shape,
                                     kv_shape, qkv_shape, q_tile, kv_tile)

        def kern():
            # the launches the step above makes
            if fused:
                return _lib.fna_backward_fused(qd, kd, vd, d_out, lse, delta, kernel, stride, dilation, causal,
                                               D**-0.5, q_tile, kv_tile)
            return kern_permuted()

        def timed(fn):
            for _ in range(2):
                fn()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(args.steps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / args.steps

        kernel_ms = timed(kern)
        kernel_permuted_ms = timed(kern_permuted)
    fwd_flops = 4.0 * B * H * D * count_attended(layout, kernel, stride, dilation, causal)
    achieved = 2.5 * fwd_flops / (kernel_ms * 1e-3) / 1e12
    peak = PEAK_TFLOPS[dt_name]
    print(json.dumps({
        "metric": "FNA fwd+bwd ms per step and effective TFLOP/s of the backward kernels, 1 GPU",
        "value": 3.5 * fwd_flops / (ms_per_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dt_name,
        "data": "synthetic",
        "config": {
            "workload": WORKLOAD_NAMES[args.workload] + ", forward + backward",
            "backward_q_tile_shape": list(q_tile),
            "backward_kv_tile_shape": list(kv_tile),
            "path": ("forward (one launch) + delta + dQ kernel + dK/dV kernel on the original tensors" if fused else
                     "forward + delta + token permutes + dQ and dK/dV kernels + unpermutes"),
        },
        "na_flop_per_step": 3.5 * fwd_flops,
        "backward_kernels_ms": kernel_ms,
        "backward_kernels_on_permuted_operands_ms": kernel_permuted_ms,
        "roofline": {
            "kernel": "fna_bwd_kernel (dQ role + dK/dV role)",
            "bound": "mfma",
            "achieved": achieved,
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": achieved / peak,
            "traffic": MEASURED_BACKWARD_TRAFFIC_BYTES.get((args.workload, tuple(q_tile), tuple(kv_tile))),
            "algorithmic_flop": 2.5 * fwd_flops,
        },
        "cpu_baseline": None,
    }), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c4", choices=sorted(WORKLOADS))
    ap.add_argument("--q-tile", type=str, default=None, help="comma separated, e.g. 2,8,8")
    ap.add_argument("--kv-tile", type=str, default=None)
    ap.add_argument("--backward", action="store_true",
                    help="measure the backward pass (forward + backward step, backward kernels) instead of the forward metric")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-mfma-probe", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus above 1 is not supported (no multi-GPU path).",
              file=sys.stderr)
        sys.exit(2)

    import torch

    import natten_amd
    from natten_amd import _lib
    from natten_amd.tile_config import check_fna_forward_config

    _lib.lib()  # no fallback: fail here when the HIP library is missing
    dev = torch.device("cuda:0")
    B, H, layout, D, kernel, stride, dilation, causal, dt_name, std = WORKLOADS[args.workload]
    quantised = dt_name == "e4m3"
    dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "e4m3": torch.bfloat16}[dt_name]
    n = len(layout)
    gen = torch.Generator().manual_seed(0)
    q, k, v = ((torch.randn((B, *layout, H, D), generator=gen) * std).to(dev) for _ in range(3))
    scales = {}
    q8 = k8 = v8 = None
    if quantised:
        # per-head absmax scaling into the e4m3 range (max finite value 448)
        def quantise(x):
            sc = x.abs().amax(dim=tuple(range(x.dim() - 2)) + (x.dim() - 1,)).float() / 448.0
            return (x / sc.view(-1, 1)).to(torch.float8_e4m3fn), sc

        (q8, sq), (k8, sk), (v8, sv) = quantise(q), quantise(k), quantise(v)
        scales = {"q_scale": sq, "k_scale": sk, "v_scale": sv, "out_dtype": torch.bfloat16}
        # the dequantised values are what the result is checked against
        q, k, v = (x8.float() * sc.view(-1, 1) for x8, sc in ((q8, sq), (k8, sk), (v8, sv)))
    else:
        q, k, v = (x.to(dtype) for x in (q, k, v))
    na = {1: natten_amd.na1d, 2: natten_amd.na2d, 3: natten_amd.na3d}[n]
    if args.backward:
        # --q-tile / --kv-tile then name the backward tiles; the forward of the step uses its defaults
        if quantised:
            print("bench.py: there is no backward pass for 8-bit float operands.", file=sys.stderr)
            sys.exit(2)
        bench_backward(args, q, k, v, kernel, stride, dilation, causal, dt_name)
        return

    q_tile = tuple(int(x) for x in args.q_tile.split(",")) if args.q_tile else None
    kv_tile = tuple(int(x) for x in args.kv_tile.split(",")) if args.kv_tile else None
    q_tile, kv_tile = check_fna_forward_config(q, kernel, stride, dilation, causal, q_tile, kv_tile)

    def step():
        if quantised:
            return na(q8, k8, v8, kernel, stride, dilation, causal, q_tile_shape=q_tile, kv_tile_shape=kv_tile,
                      return_lse=True, **scales)
        return na(q, k, v, kernel, stride, dilation, causal, q_tile_shape=q_tile, kv_tile_shape=kv_tile,
                  return_lse=True)

    with torch.no_grad():
        for _ in range(args.warmup):
            out, lse = step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out, lse = step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    flops = 4.0 * B * H * D * count_attended(layout, kernel, stride, dilation, causal)
    tflops_e2e = flops / (ms_per_step * 1e-3) / 1e12

    # ---- kernel-only timings with HIP events on the launch stream ----------------------------
    from natten_amd.token_permute import token_permute_operation, token_unpermute_operation

    with torch.no_grad():
        if quantised:
            qp, qkv_shape, q_shape = token_permute_operation(q8, q_tile, dilation)
            kp, _, kv_shape = token_permute_operation(k8, kv_tile, dilation)
            vp, _, _ = token_permute_operation(v8, kv_tile, dilation)
            kscales = {key: scales[key] for key in ("q_scale", "k_scale", "v_scale")}
            tp_in = q8
        else:
            qp, qkv_shape, q_shape = token_permute_operation(q, q_tile, dilation)
            kp, _, kv_shape = token_permute_operation(k, kv_tile, dilation)
            vp, _, _ = token_permute_operation(v, kv_tile, dilation)
            kscales = {}
            tp_in = q
        scale = D**-0.5

        fused = _lib.fused_layout_supported(layout, dilation, kv_tile)

        def kern_permuted():
            return _lib.fna_forward(qp, kp, vp, kernel, stride, dilation, causal, scale, q_shape, kv_shape,
                                    qkv_shape, q_tile, kv_tile, **kscales)

        def kern():
            # the launch the step above makes
            if fused and quantised:
                return _lib.fna_forward_fused(q8, k8, v8, kernel, stride, dilation, causal, scale, q_tile, kv_tile,
                                              **kscales)
            if fused:
                return _lib.fna_forward_fused(q, k, v, kernel, stride, dilation, causal, scale, q_tile, kv_tile)
            return kern_permuted()

        def timed(fn, iters):
            for _ in range(3):
                fn()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / iters

        kernel_ms = timed(kern, args.steps)
        kernel_permuted_ms = timed(kern_permuted, args.steps)
        op, lp = kern_permuted()
        perm_ms = timed(lambda: token_permute_operation(tp_in, q_tile, dilation), args.steps)
        unperm_ms = timed(lambda: token_unpermute_operation(op, qkv_shape, q_tile, dilation), args.steps)
    q_bytes = qp.numel() * qp.element_size()
    achieved = flops / (kernel_ms * 1e-3) / 1e12
    peak = PEAK_TFLOPS[dt_name]
    dense_flops = 4.0 * B * H * D * float(q.numel() // (B * H * D)) ** 2

    result = {
        "metric": "FNA fwd ms + effective TFLOP/s (% MFMA peak), na3d bf16 D=128, 1 GPU",
        "value": tflops_e2e,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dt_name,
        "data": "synthetic",
        "config": {
            "workload": WORKLOAD_NAMES[args.workload],
            "q_tile_shape": list(q_tile),
            "kv_tile_shape": list(kv_tile),
            "path": ("one launch: fused FNA kernel gathering tiles from the original tensors" if fused else
                     "token permute (Q,K,V) + fused FNA kernel + token unpermute (O, LSE)"),
        },
        "na_flop_per_step": flops,
        "dense_over_na_flop": dense_flops / flops,
        "kernel_ms": kernel_ms,
        "kernel_on_permuted_operands_ms": kernel_permuted_ms,
        "token_permute": {
            "permute_q_ms": perm_ms,
            "unpermute_o_ms": unperm_ms,
            "permute_GBps": 2 * q_bytes / (perm_ms * 1e-3) / 1e9,
            "unpermute_GBps": 2 * op.numel() * op.element_size() / (unperm_ms * 1e-3) / 1e9,
        },
        "roofline": {
            "kernel": "fna_fwd_fp8_kernel" if quantised else "fna_fwd_kernel",
            "bound": "mfma",
            "achieved": achieved,
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": achieved / peak,
            "traffic": MEASURED_TRAFFIC_BYTES.get((args.workload, tuple(q_tile), tuple(kv_tile))),
            "algorithmic_bytes": (4 * q.numel() * (1 if quantised else q.element_size())
                                  + (q.numel() if quantised else 0) + lse.numel() * 4),
        },
    }
    if not args.no_mfma_probe:
        # context for roofline.frac: what the matrix cores sustain on random operands under the
        # chip's power limit (the published peak assumes the maximum clock)
        rnd_tflops, rnd_ghz = _lib.mfma_probe(random_operands=True)
        const_tflops, const_ghz = _lib.mfma_probe(random_operands=False)
        result["mfma_probe"] = {
            "instruction": "v_mfma_f32_32x32x16_bf16, one wave per SIMD, nothing else",
            "random_operands": {"TFLOP/s": rnd_tflops, "shader_clock_GHz": rnd_ghz},
            "constant_operands": {"TFLOP/s": const_tflops, "shader_clock_GHz": const_ghz},
        }
    if not args.no_cpu_baseline:
        # 16-bit operands: atol = rtol = 1e-2; 8-bit matrix path (P rounded to e4m3, relative error
        # up to 2^-4 per probability): atol = rtol = 2^-4
        result["cpu_baseline"] = cpu_baseline(q, k, v, kernel, stride, dilation, causal, out, lse,
                                              tol=2.0**-4 if quantised else 1e-2)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
