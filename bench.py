"""Benchmark of the MI355X neighborhood attention forward path.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4|c3|c2|c2d]

One step = one na3d/na2d forward through the public API on inputs already resident in HBM:
a single launch that gathers its tiles from the original tensors when the problem allows it
(all benchmark workloads do), else token permute of Q/K/V, kernel, unpermute of O and LSE.  Prints ONE JSON line: whole-path throughput in effective
NA TFLOP/s (4 * B * H * D * sum_q |window(q)| per step), the fused kernel's roofline figures from
HIP events over the timed steps, and a CPU baseline: the PyTorch call the reference's CPU path makes
(flex_attention with the neighborhood block mask, oracle/flex_cpu.py) timed on this box's host
cores, on the workload itself where the dense N x N mask fits in memory and on a labelled cropped
proxy where it does not; the C oracle's rate on a sample of the workload's queries is reported
beside it (and checks the GPU result on that sample).
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
HBM_PEAK_GBPS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "e4m3": 5000.0, "fp32": 157.3}

WORKLOADS = {
    # name: (B, H, layout, D, kernel, stride, dilation, causal, dtype, std)
    "c4": (1, 24, (30, 48, 80), 128, (18, 24, 24), (1, 8, 8), (1, 1, 1), (True, False, False), "bf16", 1.0),
    "c3": (1, 16, (128, 128), 128, (32, 32), (16, 16), (1, 1), (False, False), "fp16", 0.5),
    "c2": (2, 8, (64, 64), 64, (13, 13), (1, 1), (1, 1), (False, False), "bf16", 1.0),
    "c2d": (2, 8, (64, 64), 64, (13, 13), (1, 1), (2, 2), (False, False), "bf16", 1.0),
    # the configuration the reference runs on the CPU, at its stated type (the float32 kernel, token-permuted route)
    "c1": (1, 2, (256,), 32, (7,), (1,), (1,), (False,), "fp32", 1.0),
    # e4m3 operands with per-head absmax scales, bf16 output; multiplied by the 8-bit matrix instruction
    "c5": (1, 16, (16, 64, 64), 128, (8, 16, 16), (4, 8, 8), (1, 2, 2), (False, False, False), "e4m3", 1.0),
    # the shapes the reference publishes runtimes for (docs/profiler.md:853-876, :925-951, :654-755; fp16, batch 1)
    "hunyuan_na": (1, 24, (30, 48, 80), 128, (18, 24, 24), (1, 1, 1), (1, 1, 1), (False, False, False), "fp16", 1.0),
    "hunyuan_gna": (1, 24, (30, 48, 80), 128, (18, 24, 24), (16, 8, 8), (1, 1, 1), (False, False, False), "fp16", 1.0),
    "flux_na": (1, 24, (256, 256), 128, (80, 80), (1, 1), (1, 1), (False, False), "fp16", 1.0),
    "flux_gna": (1, 24, (256, 256), 128, (80, 80), (16, 16), (1, 1), (False, False), "fp16", 1.0),
    # its 1-D use case (docs/profiler.md:325-560; one head, 32K tokens, 2K window: sliding, strided, blocked)
    "na1d_32k": (1, 1, (32768,), 128, (2048,), (1,), (1,), (False,), "fp16", 1.0),
    "na1d_32k_s256": (1, 1, (32768,), 128, (2048,), (256,), (1,), (False,), "fp16", 1.0),
    "na1d_32k_blocked": (1, 1, (32768,), 128, (2048,), (2048,), (1,), (False,), "fp16", 1.0),
    # extents that no tile shape divides (and an uneven dilation in time): the one-launch route clamps
    # its gathers; compare `ms_per_step` with `e2e_permuted_route_ms`
    "odd3d": (1, 24, (29, 46, 78), 128, (9, 24, 24), (1, 8, 8), (2, 1, 1), (False, False, False), "bf16", 1.0),
}
# Published forward runtimes of the reference's Blackwell FNA kernel on a B200 for those shapes
# (kernel only / with token permute; docs/sample-outputs/profiler-*-blackwell-fna-b200.txt): other
# hardware, context only, never a baseline for `vs_baseline`.
SUB_MILLISECOND_WORKLOADS = ("c1", "c2", "c2d", "c3", "c5", "na1d_32k", "na1d_32k_s256", "na1d_32k_blocked")

REFERENCE_B200_MS = {
    "hunyuan_na": (42.243, 47.353),
    "hunyuan_gna": (13.010, 18.538),
    "flux_na": (8.692, 10.931),
    "flux_gna": (4.114, 6.389),
    # (1-D, dilation 1: the reference launches its kernel on the tensors as they are)
    "na1d_32k": (0.058111, 0.058111),
    "na1d_32k_s256": (0.037888, 0.037888),
    "na1d_32k_blocked": (0.038240, 0.038240),
}
# Cropped proxies for the CPU baseline where the reference's CPU path (dense N x N mask and scores)
# does not fit in memory: same kernel / stride / dilation / causal / head dim on a smaller layout
# and fewer heads.  name -> (layout, heads); workloads not listed run as they are (c3: one head at a time).
CPU_PROXY = {
    "c4": ((20, 24, 24), 2),
    "c5": ((8, 32, 32), 2),
    "hunyuan_na": ((20, 24, 24), 2),
    "hunyuan_gna": ((20, 24, 24), 2),
    "flux_na": ((96, 96), 2),
    "flux_gna": ((96, 96), 2),
    "odd3d": ((19, 25, 27), 2),
    "na1d_32k": ((8192,), 1),
    "na1d_32k_s256": ((8192,), 1),
    "na1d_32k_blocked": ((8192,), 1),
}
# HBM-side traffic of a launch (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, calibrated on a copy of known
# size) is read from the profile summaries, which carry one line per measurement:
#   traffic: workload=c4 pass=forward q_tile=2,8,8 kv_tile=1,8,8 bytes=2.82e10 kernel_digest=<hex>
# and is reported only while `kernel_digest` equals the digest of the kernel sources this run uses;
# after any change to those sources the bench prints null until the counters are collected again.
KERNEL_SOURCES = {
    # kernels and launch geometry of each pass (the C entry points around them do not touch the traffic)
    "forward": ["fna_fwd.hpp", "na_math.hpp"],
    "forward_fp8": ["fna_fwd.hpp", "fna_fwd_fp8.hpp", "na_math.hpp"],
    "backward": ["fna_fwd.hpp", "fna_bwd.hpp", "na_math.hpp"],
}


def kernel_digest(which="forward"):
    import hashlib

    h = hashlib.sha256()
    for name in KERNEL_SOURCES[which]:
        with open(os.path.join(ROOT, "natten_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload, which, q_tile, kv_tile):
    """Bytes per launch from profiles/*.md for this workload, pass and tiles, or None when no
    measurement of the current kernel sources is on file."""
    import glob
    import re

    want = {"workload": workload, "pass": which, "q_tile": ",".join(map(str, q_tile)),
            "kv_tile": ",".join(map(str, kv_tile)), "kernel_digest": kernel_digest(which)}
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.md"))):
        with open(path) as f:
            for line in f:
                if not line.lstrip().startswith("traffic:"):
                    continue
                kv = dict(re.findall(r"(\w+)=(\S+)", line))
                if all(kv.get(key) == val for key, val in want.items()) and "bytes" in kv:
                    return {"bytes": float(kv["bytes"]), "source": os.path.relpath(path, ROOT)}
    return None


WORKLOAD_NAMES = {
    "c4": "na3d bf16 B=1 H=24 30x48x80 D=128 k=(18,24,24) s=(1,8,8) causal=(T,F,F) +LSE",
    "c3": "na2d fp16 B=1 H=16 128x128 D=128 k=(32,32) s=(16,16)",
    "c1": "na1d fp32 B=1 H=2 L=256 D=32 k=7",
    "c2": "na2d bf16 B=2 H=8 64x64 D=64 k=(13,13)",
    "c2d": "na2d bf16 B=2 H=8 64x64 D=64 k=(13,13) d=(2,2)",
    "c5": "na3d e4m3 (per-head scales, bf16 out) B=1 H=16 16x64x64 D=128 k=(8,16,16) s=(4,8,8) d=(1,2,2)",
    "hunyuan_na": "na3d fp16 B=1 H=24 30x48x80 D=128 k=(18,24,24)",
    "hunyuan_gna": "na3d fp16 B=1 H=24 30x48x80 D=128 k=(18,24,24) s=(16,8,8)",
    "flux_na": "na2d fp16 B=1 H=24 256x256 D=128 k=(80,80)",
    "flux_gna": "na2d fp16 B=1 H=24 256x256 D=128 k=(80,80) s=(16,16)",
    "odd3d": "na3d bf16 B=1 H=24 29x46x78 D=128 k=(9,24,24) s=(1,8,8) d=(2,1,1)",
    "na1d_32k": "na1d fp16 B=1 H=1 L=32768 D=128 k=2048",
    "na1d_32k_s256": "na1d fp16 B=1 H=1 L=32768 D=128 k=2048 s=256",
    "na1d_32k_blocked": "na1d fp16 B=1 H=1 L=32768 D=128 k=2048 s=2048",
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


def c_oracle_sample(q, k, v, kernel, stride, dilation, causal, out_gpu, lse_gpu, seconds_target=6.0, tol=1e-2):
    """C oracle on a bounded sample of this workload's queries (all heads) on the host cores: its
    rate, and the GPU result checked against it on that sample."""
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
        "sample": f"C oracle (float64 window walk), {nq} random queries x {H} heads of this workload, {dt:.1f} s wall",
        "gpu_parity_on_sample": {"ok": ok, "max_abs_err_out": err_o, "max_abs_err_lse": err_l, "atol_rtol": tol},
    }


def cpu_baseline(workload, q, k, v, kernel, stride, dilation, causal, dt_name, std, timed_runs=2):
    """The reference's CPU path, timed on this box's host cores: torch.nn.attention.flex_attention
    with the neighborhood block mask on CPU tensors (the one PyTorch call `flex_fna_generic` makes
    without tile shapes, src/natten/backends/flex.py:126-137, :538-547; restated in
    oracle/flex_cpu.py).  Eager flex on the CPU materialises N x N masks and scores: the workload
    runs as it is when that fits, one head at a time when only that fits, and otherwise the call is
    reported as not fitting and a cropped proxy (same window parameters, smaller layout, two heads)
    is timed instead, labelled as such, and checked against the C oracle."""
    import warnings

    import numpy as np
    import torch

    from oracle import c_oracle
    from oracle.flex_cpu import flex_na_cpu

    B, H, D = q.shape[0], q.shape[-2], q.shape[-1]
    n = q.dim() - 3
    layout = tuple(int(x) for x in q.shape[1 : 1 + n])
    N = int(np.prod(layout))
    cpu_dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "e4m3": torch.bfloat16, "fp32": torch.float32}[dt_name]
    info = {"unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "call": "torch.nn.attention.flex_attention + create_block_mask(BLOCK_SIZE=(64, 64), device='cpu') on "
                    "[B, H, N, D] CPU tensors, return_lse=True, FORCE_USE_FLEX_ATTENTION: the call of the reference's "
                    "CPU path (flex-fna backend), with its mask_mod restated",
            "os_cpu_count": os.cpu_count(), "torch_num_threads": torch.get_num_threads()}
    proxy = CPU_PROXY.get(workload)
    if proxy is not None:
        p_layout, p_heads = proxy
        info["fits"] = False
        info["reason"] = (f"N = {N} tokens: the dense N x N boolean mask alone is {N * N / 1e9:.1f} GB and the float32 "
                          f"scores {4.0 * N * N / 1e9:.1f} GB per head")
        gen = torch.Generator().manual_seed(0)
        cq, ck, cv = ((torch.randn((1, *p_layout, p_heads, D), generator=gen) * std).to(cpu_dtype) for _ in range(3))
        heads_timed, layout_timed = p_heads, p_layout
        sample = (f"cropped proxy: same kernel_size / stride / dilation / is_causal / head_dim on "
                  f"{'x'.join(map(str, p_layout))}, B=1, H={p_heads}, {cpu_dtype}".replace("torch.", ""))
    else:
        info["fits"] = True
        per_head = N > 8192  # float32 scores of all heads at once would not fit: one head per call
        cq, ck, cv = (t[:1].to("cpu", cpu_dtype) for t in (q, k, v)) if per_head else (t.to("cpu", cpu_dtype) for t in (q, k, v))
        if per_head:
            cq, ck, cv = (t[..., :1, :].contiguous() for t in (cq, ck, cv))
        heads_timed, layout_timed = cq.shape[-2], layout
        sample = ("the workload itself" if not per_head else
                  f"the workload one head at a time: 1 of {B * H} (batch, head) pairs timed")
    attended = count_attended(layout_timed, kernel, stride, dilation, causal)
    flops = 4.0 * cq.shape[0] * heads_timed * D * attended
    times = []
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        with torch.no_grad():
            for i in range(1 + timed_runs):  # first run untimed: warm-up
                t0 = time.perf_counter()
                ref_out, ref_lse = flex_na_cpu(cq, ck, cv, kernel, stride, dilation, causal)
                if i:
                    times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    info["value"] = flops / med / 1e12
    info["seconds_per_call"] = med
    info["sample"] = f"{sample}; 1 warm-up + {timed_runs} timed calls, median"
    # the flex result against the C oracle on the same inputs (rows of the first head pair)
    rng = np.random.default_rng(1)
    Np = int(np.prod(layout_timed))
    tok = rng.integers(0, Np, size=64)
    o_ref, l_ref, _ = c_oracle.na_rows(cq.float().numpy(), ck.float().numpy(), cv.float().numpy(), kernel, stride,
                                       dilation, causal, None, np.zeros(64, dtype=np.int32), tok, 8)
    got_o = ref_out.reshape(cq.shape[0], Np, heads_timed, D)[0, torch_idx(tok)].float().numpy()
    got_l = ref_lse.reshape(cq.shape[0], Np, heads_timed)[0, torch_idx(tok)].float().numpy()
    info["flex_vs_c_oracle"] = {"max_abs_err_out": float(np.abs(got_o - o_ref).max()),
                                "max_abs_err_lse": float(np.abs(got_l - l_ref).max())}
    return info


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
    tiles_given = q_tile is not None
    q_tile, kv_tile = check_fna_backward_config(q, kernel, stride, dilation, causal, q_tile, kv_tile)
    gen = torch.Generator().manual_seed(1)
    d_out = torch.randn(q.shape, generator=gen).to(q.dtype).to(q.device)
    q, k, v = (t.clone().requires_grad_(True) for t in (q, k, v))

    def step():
        q.grad = k.grad = v.grad = None
        out = na(q, k, v, kernel, stride, dilation, causal, backward_q_tile_shape=q_tile if tiles_given else None,
                 backward_kv_tile_shape=kv_tile if tiles_given else None)
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
        # left to itself the op gives each launch on the original tensors the tile shapes that suit its role
        kv_role = (None, None)
        if fused and not tiles_given:
            from natten_amd.tile_config import choose_backward_role_tile_shapes

            roles = choose_backward_role_tile_shapes(layout, tuple(kernel), tuple(stride), tuple(dilation), tuple(causal))
            if roles is not None and all(_lib.backward_fused_layout_supported(layout, dilation, a, b) for a, b in roles):
                (q_tile_dq, kv_tile_dq), kv_role = roles
            else:
                q_tile_dq, kv_tile_dq = q_tile, kv_tile
        else:
            q_tile_dq, kv_tile_dq = q_tile, kv_tile

        def kern_permuted():
            return _lib.fna_backward(qp, kp, vp, dop, lp, dp, kernel, stride, dilation, causal, D**-0.5, q_shape,
                                     kv_shape, qkv_shape, q_tile, kv_tile)

        def kern():
            # the launches the step above makes
            if fused:
                return _lib.fna_backward_fused(qd, kd, vd, d_out, lse, delta, kernel, stride, dilation, causal,
                                               D**-0.5, q_tile_dq, kv_tile_dq, *kv_role)
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

        # (--step-only: the step's launches alone, for profiles; the rate then counts the whole step's time)
        kernel_ms = None if args.step_only else timed(kern)
        kernel_permuted_ms = None if args.step_only else timed(kern_permuted)
    fwd_flops = 4.0 * B * H * D * count_attended(layout, kernel, stride, dilation, causal)
    achieved = 2.5 * fwd_flops / ((kernel_ms if kernel_ms is not None else ms_per_step) * 1e-3) / 1e12
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
            "backward_q_tile_shape": list(q_tile_dq),
            "backward_kv_tile_shape": list(kv_tile_dq),
            "dk_dv_launch_tile_shapes": [list(t) for t in kv_role] if kv_role[0] is not None else None,
            "permuted_route_tile_shapes": [list(q_tile), list(kv_tile)],
            "path": ("forward (one launch) + delta + scaled queries + dK/dV kernel + dQ kernel on the original tensors" if fused else
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
            "traffic": (measured_traffic(args.workload, "backward", q_tile_dq, kv_tile_dq) or {}).get("bytes"),
            "kernel_digest": kernel_digest("backward"),
            "algorithmic_flop": 2.5 * fwd_flops,
        },
        "cpu_baseline": None,
    }), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps (default 20; 300 for the workloads whose step takes less than a millisecond)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default 5; 100 for those)")
    ap.add_argument("--workload", default="c4", choices=sorted(WORKLOADS))
    ap.add_argument("--q-tile", type=str, default=None, help="comma separated, e.g. 2,8,8")
    ap.add_argument("--kv-tile", type=str, default=None)
    ap.add_argument("--backward", action="store_true",
                    help="measure the backward pass (forward + backward step, backward kernels) instead of the forward metric")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--step-only", action="store_true",
                    help="skip the side measurements (kernel through the C ABI alone, token-permuted route): "
                         "a profile of such a run holds the step's launches only")
    ap.add_argument("--no-mfma-probe", action="store_true")
    ap.add_argument("--no-dense", action="store_true",
                    help="skip the dense self-attention run of the same tensors (measured speed-up against the FLOP ratio)")
    args = ap.parse_args()
    # a step of the small workloads lasts 30-200 us: twenty of them end before the device's clocks have
    # settled (c3 reads 0.19-0.21 ms over 20 steps and 0.162 ms sustained), so they get longer loops
    short = args.workload in SUB_MILLISECOND_WORKLOADS and not args.backward
    if args.steps is None:
        args.steps = 300 if short else 20
    if args.warmup is None:
        args.warmup = 100 if short else 5
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
    dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "e4m3": torch.bfloat16, "fp32": torch.float32}[dt_name]
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

    # One loop gives both figures: the host clock around the K steps (bracketed by synchronisation)
    # and HIP events recorded on the launch stream (torch's current stream) before the first and
    # after the last of the same K steps.
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    with torch.no_grad():
        for _ in range(args.warmup):
            out, lse = step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev0.record()
        for _ in range(args.steps):
            out, lse = step()
        ev1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    step_events_ms = ev0.elapsed_time(ev1) / args.steps
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

        # (float32 operands have no one-launch form: their step is permute + kernel + unpermute)
        fused = dtype != torch.float32 and _lib.fused_layout_supported(layout, dilation, kv_tile, q_tile_shape=q_tile,
                                                                       dtype=None if quantised else dtype)

        from natten_amd.functional import work_queue_default

        # the launch kind the public call above picked (work queue or a workgroup per Q tile)
        kscales["run_persistent"] = work_queue_default(B, H, layout, kernel, stride, dilation, causal, q_tile, kv_tile)

        def kern_permuted():
            return _lib.fna_forward(qp, kp, vp, kernel, stride, dilation, causal, scale, q_shape, kv_shape,
                                    qkv_shape, q_tile, kv_tile, **kscales)

        def kern():
            # the launch the step above makes
            if fused and quantised:
                return _lib.fna_forward_fused(q8, k8, v8, kernel, stride, dilation, causal, scale, q_tile, kv_tile,
                                              **kscales)
            if fused:
                return _lib.fna_forward_fused(q, k, v, kernel, stride, dilation, causal, scale, q_tile, kv_tile,
                                              **kscales)
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

        # the step is this one launch when the one-launch route applies: its duration is then the
        # event time of the timed steps themselves; otherwise the kernel is timed on its own
        kernel_ms = step_events_ms if fused else timed(kern, args.steps)
        extras = {}
        if not args.step_only:
            kernel_alone_ms = timed(kern, args.steps)
            kernel_permuted_ms = timed(kern_permuted, args.steps)
            op, lp = kern_permuted()
            perm_ms = timed(lambda: token_permute_operation(tp_in, q_tile, dilation), args.steps)
            unperm_ms = timed(lambda: token_unpermute_operation(op, qkv_shape, q_tile, dilation), args.steps)
            q_bytes = qp.numel() * qp.element_size()
            extras = {
                "kernel_direct_call_ms": kernel_alone_ms,
                "kernel_on_permuted_operands_ms": kernel_permuted_ms,
                "e2e_permuted_route_ms": 3 * perm_ms + kernel_permuted_ms + unperm_ms,
                "token_permute": {
                    "permute_q_ms": perm_ms,
                    "unpermute_o_ms": unperm_ms,
                    "permute_GBps": 2 * q_bytes / (perm_ms * 1e-3) / 1e9,
                    "unpermute_GBps": 2 * op.numel() * op.element_size() / (unperm_ms * 1e-3) / 1e9,
                },
            }
    achieved = flops / (kernel_ms * 1e-3) / 1e12
    peak = PEAK_TFLOPS[dt_name]
    from natten_amd.tile_config import visited_pairs

    attended = B * H * count_attended(layout, kernel, stride, dilation, causal)
    visited = B * H * visited_pairs(layout, kernel, stride, dilation, causal, q_tile, kv_tile, anchored=bool(fused))
    dense_flops = 4.0 * B * H * D * float(q.numel() // (B * H * D)) ** 2

    # bytes of Q, K, V read and O, LSE written once
    alg_bytes = (4 * q.numel() * (1 if quantised else q.element_size()) + (q.numel() if quantised else 0)
                 + q.numel() // D * 4)
    which = "forward_fp8" if quantised else "forward"
    traffic = measured_traffic(args.workload, which, q_tile, kv_tile) if fused else None
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
            "launch": "work queue (resident workgroups pull Q tiles)" if kscales["run_persistent"] else "one workgroup per Q tile",
        },
        "na_flop_per_step": flops,
        "dense_over_na_flop": dense_flops / flops,
        # (query, key) pairs the kernel multiplies (whole tiles of the KV box of every Q tile, padding
        # included) against the pairs the neighborhood holds: the geometric waste of the tiling
        "visited_pairs": visited,
        "attended_pairs": attended,
        "visited_over_attended": visited / attended,
        "kernel_ms": kernel_ms,
        "kernel_ms_source": ("HIP events around the timed steps (one launch per step)" if fused else
                             "HIP events around kernel-only launches"),
        **extras,
        "roofline": {
            "kernel": ("fna_fwd_f32_kernel" if dtype == torch.float32 else
                       ("fna_fwd_fp8" if quantised else "fna_fwd") +
                       ("_queue_kernel" if kscales["run_persistent"] else "_kernel")),
            "bound": "mfma",
            "achieved": achieved,
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": achieved / peak,
            "traffic": traffic["bytes"] if traffic else None,
            "traffic_source": traffic["source"] if traffic else None,
            "kernel_digest": kernel_digest(which),
            "algorithmic_bytes": alg_bytes,
        },
    }
    if flops / alg_bytes < peak * 1e12 / (HBM_PEAK_GBPS * 1e9):
        # fewer FLOP per algorithmic byte than the chip's ridge point: memory (here mostly launch latency) bounds
        # the kernel, and the figure to read is bytes per second (c1, c2)
        gbps = alg_bytes / (kernel_ms * 1e-3) / 1e9
        result["roofline"].update({"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                   "frac": gbps / HBM_PEAK_GBPS, "mfma_frac": achieved / peak})
    if not args.no_dense and not args.step_only and dtype != torch.float32:
        # The other half of the comparison the reference publishes per shape (docs/profiler.md:837-876:
        # measured speed-up over self attention beside the FLOP-wise upper bound): dense attention over the
        # same tokens, flattened to one sequence, through this library's own dense kernel.
        N = q.numel() // (B * H * D)
        flat = lambda t: t.reshape(B, N, H, D)
        with torch.no_grad():
            if quantised:
                dense = lambda: natten_amd.attention(flat(q8), flat(k8), flat(v8), **scales)
            else:
                dense = lambda: natten_amd.attention(flat(q), flat(k), flat(v))
            dense_iters = max(2, min(args.steps, int(0.5 / max(kernel_ms * 1e-3 * dense_flops / flops, 1e-6))))
            dense_ms = timed(dense, dense_iters)
        result["dense_self_attention"] = {
            "call": "natten_amd.attention on the same tensors as one sequence of %d tokens" % N,
            "dense_ms": dense_ms,
            "dense_TFLOPs": dense_flops / (dense_ms * 1e-3) / 1e12,
            "timed_calls": dense_iters,
            "measured_speedup_vs_dense": dense_ms / kernel_ms,
            "flop_wise_upper_bound": dense_flops / flops,
            "fraction_of_bound": (dense_ms / kernel_ms) / (dense_flops / flops),
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
        result["cpu_baseline"] = cpu_baseline(args.workload, q, k, v, kernel, stride, dilation, causal, dt_name, std)
        result["cpu_baseline"]["c_oracle"] = c_oracle_sample(q, k, v, kernel, stride, dilation, causal, out, lse,
                                                             tol=2.0**-4 if quantised else 1e-2)
    if args.workload in REFERENCE_B200_MS:
        ref_k, ref_e2e = REFERENCE_B200_MS[args.workload]
        result["reference_published_b200"] = {
            "kernel_ms": ref_k, "with_token_permute_ms": ref_e2e,
            "note": "the reference's Blackwell FNA kernel on an NVIDIA B200 (its docs/profiler.md): other hardware, context only"}
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
