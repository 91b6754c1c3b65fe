#!/usr/bin/env python3
"""Benchmark of the FLARE mixer forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one forward of the mixer (split-N gather, merge, scatter) over the headline workload
B=1, H=8, N=1,048,576, M=256, D=32, bf16 in / fp32 accumulate, inputs resident in HBM.
Prints ONE JSON line: tokens/s, the roofline of the dominant kernel (measured with HIP events
on the launch stream), and the CPU baseline (torch SDPA, MATH backend, fp32) timed on this
machine's host cores on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published


def make_inputs(B, H, N, M, D, dtype, device, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    q = (torch.randn(H, M, D, generator=g) * D ** -0.5).to(dtype)
    gk = torch.Generator(device=device).manual_seed(seed)
    k = torch.randn(B, H, N, D, generator=gk, device=device, dtype=torch.float32).to(dtype)
    v = torch.randn(B, H, N, D, generator=gk, device=device, dtype=torch.float32).to(dtype)
    return q.to(device), k, v


def time_events(fn, steps, warmup):
    """Average duration (ms) of fn() over `steps` calls, HIP events on the current stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def copy_bandwidth(device):
    """Measured streaming-copy GB/s (read + write) of a 1 GiB buffer, for orientation."""
    a = torch.empty(1 << 28, dtype=torch.float32, device=device)
    b = torch.empty_like(a)
    ms = time_events(lambda: b.copy_(a), 10, 3)
    return 2 * a.numel() * 4 / (ms * 1e-3) / 1e9


def cpu_baseline(q, k, v, n_sample):
    """Reference CPU path: y = SDPA(k, q, SDPA(q, k, v)), MATH backend, fp32, per head."""
    from oracle import flare_oracle as O

    qc = q.float().cpu()
    kc = k[:, :, :n_sample].float().cpu()
    vc = v[:, :, :n_sample].float().cpu()
    H = kc.shape[1]
    outs = []
    t0 = time.perf_counter()
    for h in range(H):
        y, _ = O.mixer_sdpa(qc[h : h + 1], kc[:, h : h + 1], vc[:, h : h + 1], 1.0)
        outs.append(y)
    dt = time.perf_counter() - t0
    return torch.cat(outs, dim=1), dt


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--cpu-sample", type=int, default=1048576, help="tokens of the CPU baseline sample")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this build has no multi-GPU path (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        sys.exit(1)

    import flare_py_amd as F

    dev = torch.device("cuda:0")
    B, H, N, M, D = 1, 8, 1 << 20, 256, 32
    dtype = torch.bfloat16
    q, k, v = make_inputs(B, H, N, M, D, dtype, dev)
    kernel = F.mixer_kernel_name(q, k, v)

    # ---- whole step, wall clock between device synchronisations -------------------------
    step = lambda: F.flare_multihead_mixer(q, k, v)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps
    tokens_per_s = B * N / (ms_step * 1e-3)

    # ---- per-kernel durations (HIP events on the launch stream) --------------------------
    z, _ = F.flare_gather(q, k, v)
    ms_gather = time_events(lambda: F.flare_gather(q, k, v), args.steps, 2)       # split-N kernel + merge
    ms_scatter = time_events(lambda: F.flare_scatter(q, k, z), args.steps, 2)
    esz = 2
    bytes_gather = 2 * B * H * N * D * esz          # K and V read once
    bytes_scatter = 2 * B * H * N * D * esz         # K read, Y written
    flops_phase = 4 * B * H * N * M * D             # per phase: two products of 2*N*M*D
    # HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two passes, scaled by the
    # readings of a 1 GiB copy: x2.000 and x1.000); they cannot be collected from inside this process.
    traffic_measured = {"gather_mfma_kernel": 1.0928e9, "scatter_mfma_kernel": 1.0770e9}
    if ms_gather >= ms_scatter:
        dom, ms_dom, bytes_dom = "gather_mfma_kernel", ms_gather, bytes_gather
    else:
        dom, ms_dom, bytes_dom = "scatter_mfma_kernel", ms_scatter, bytes_scatter
    achieved = bytes_dom / (ms_dom * 1e-3) / 1e9
    t_hbm = 4 * B * H * N * D * esz / (HBM_PEAK_GBPS * 1e9)
    t_mfma = 2 * flops_phase / (MFMA_BF16_PEAK_TFLOPS * 1e12)
    roofline = {
        "bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic_measured[dom],
        "algorithmic_bytes": bytes_dom,
        "ms_gather": round(ms_gather, 4), "ms_scatter": round(ms_scatter, 4),
        "mixer_frac_of_roofline": round(max(t_hbm, t_mfma) * 1e3 / ms_step, 4),
        "mixer_tflops": round(2 * flops_phase / (ms_step * 1e-3) / 1e12, 1),
        "mfma_peak_tflops": MFMA_BF16_PEAK_TFLOPS,
        "copy_GBps_measured": round(copy_bandwidth(dev), 1),
    }

    out = {
        "metric": "FLARE mixer tokens/sec at N=1M,M=256,D=32 bf16", "value": round(tokens_per_s, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "FLARE mixer forward B=1,H=8,N=1048576,M=256,D=32 (BASELINE config 3)",
                   "kernel": kernel, "scale": 1.0, "seed": 0},
        "roofline": roofline,
    }

    # ---- CPU baseline on a bounded sample + parity of the HIP path on the same sample ----
    if not args.no_cpu:
        ns = min(args.cpu_sample, N)
        y_cpu, dt = cpu_baseline(q, k, v, ns)
        y_gpu = F.flare_multihead_mixer(q, k[:, :, :ns], v[:, :, :ns]).float().cpu()
        rel = float((y_gpu.double() - y_cpu.double()).norm() / y_cpu.double().norm())
        out["cpu_baseline"] = {
            "value": round(B * ns / dt, 1), "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"first {ns} tokens of the same seeded workload, all {H} heads, torch SDPA MATH backend fp32, "
                      f"{dt:.2f} s",
        }
        out["rel_l2_vs_cpu_on_sample"] = rel
    print(json.dumps(out))


if __name__ == "__main__":
    main()
