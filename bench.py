#!/usr/bin/env python3
"""Benchmark of the operator hot path on one MI355X.

``python bench.py [--gpus 1] [--steps K] [--warmup W]`` prints ONE JSON line.

Headline workload (``config.workload``): ``selective_scan`` forward at the
Mamba-1 prefill shape B=8, D=1536, L=2048, N=16 with bf16 activations, fp32
state, one B/C group, D skip, z gate, dt_bias and softplus.  A "step" is one
forward pass over one batch of synthetic inputs already resident in HBM; four
input/output sets (about 0.8 GB) are rotated so that a step does not find the
previous step's data in the 256 MB last-level cache.

``value`` is algorithmic bytes per step / wall time per step (GB/s) over the K
timed steps.  ``roofline`` prices the same bytes against the kernel's own
average duration measured with HIP events on the launch stream.
``cpu_baseline`` times the CPU restatement of the reference's Python path
(``oracle/``) on a bounded slice of the same workload on this host.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def _event_ms(fn, iters):
    """Average duration (ms) of ``fn``'s GPU work, one event pair per call, on the
    current stream (the stream the kernels are launched on)."""
    pairs = []
    for i in range(iters):
        s = torch.cuda.Event(enable_timing=True)
        e = torch.cuda.Event(enable_timing=True)
        s.record()
        fn(i)
        e.record()
        pairs.append((s, e))
    torch.cuda.synchronize()
    times = sorted(s.elapsed_time(e) for s, e in pairs)
    return sum(times) / len(times), times[len(times) // 2]


def bench_scan_fwd(steps, warmup, dtype=torch.bfloat16, batch=8, dim=1536, length=2048, nstate=16,
                   nsets=4):
    from ssm_amd import configs
    from ssm_amd.ops import ScanPlan

    plans = []
    for s in range(nsets):
        inp = configs.to_device(configs.scan_inputs(batch, dim, length, nstate, dtype=dtype, seed=s))
        plans.append(ScanPlan(inp["u"], inp["delta"], inp["A"], inp["B"], inp["C"], inp["D"], inp["z"],
                              inp["dt_bias"], True, True))
    elt = 2 if dtype != torch.float32 else 4
    nbytes = configs.scan_fwd_bytes(batch, dim, length, nstate, elt)

    for i in range(warmup):
        plans[i % nsets].run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        plans[i % nsets].run()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps

    avg_ms, med_ms = _event_ms(lambda i: plans[i % nsets].run(), max(steps, 10))
    return dict(bytes=nbytes, wall_s=wall, kernel_ms=avg_ms, kernel_ms_median=med_ms,
                tokens=batch * length)


def cpu_baseline_scan(dtype=torch.bfloat16, dim=1536, length=2048, nstate=16, budget_s=15.0):
    """Time the CPU restatement of the reference's Python loop on a batch slice
    of the headline workload; returns GB/s of the same algorithmic bytes."""
    from oracle import ops_oracle
    from ssm_amd import configs

    elt = 2 if dtype != torch.float32 else 4
    batch = 1
    inp = configs.scan_inputs(batch, dim, length, nstate, dtype=dtype, seed=0)

    def once():
        t0 = time.perf_counter()
        ops_oracle.selective_scan(inp["u"], inp["delta"], inp["A"], inp["B"], inp["C"], D=inp["D"],
                                  z=inp["z"], dt_bias=inp["dt_bias"], softplus=True,
                                  return_last_state=True)
        return time.perf_counter() - t0

    first = once()
    reps = max(1, min(5, int(budget_s / max(first, 1e-3)) - 1))
    times = [first] + [once() for _ in range(reps)]
    best = sorted(times)[len(times) // 2]
    nbytes = configs.scan_fwd_bytes(batch, dim, length, nstate, elt)
    return dict(value=nbytes / best / 1e9, unit="GB/s", cores=torch.get_num_threads(), kind="port",
                sample=f"selective_scan fwd, batch slice B={batch} of the headline workload "
                       f"(D={dim}, L={length}, N={nstate}, {str(dtype).split('.')[-1]}), "
                       f"median of {len(times)} runs, {best * 1e3:.0f} ms each; "
                       f"host has {os.cpu_count()} logical cpus",
                seconds_per_call=best)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="only the headline kernel")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every operator on this path is independent per "
              "(batch, channel) row and no multi-GPU figure is defined; run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm device", file=sys.stderr)
        sys.exit(1)

    r = bench_scan_fwd(args.steps, args.warmup)
    value = r["bytes"] / r["wall_s"] / 1e9
    achieved = r["bytes"] / (r["kernel_ms"] * 1e-3) / 1e9
    line = {
        "metric": "selective_scan GB/s (%HBM peak)",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(r["wall_s"] * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "selective_scan forward, B=8 D=1536 L=2048 N=16, bf16 activations, "
                               "fp32 state, G=1 time-varying B/C, D skip, z gate, dt_bias, softplus",
                   "io_dtype": "bf16", "tokens_per_step": r["tokens"],
                   "tokens_per_s": round(r["tokens"] / r["wall_s"], 1),
                   "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "scan_fwd_kernel<bf16, 8>", "kernel_us": round(r["kernel_ms"] * 1e3, 2),
                     "algorithmic_bytes": r["bytes"]},
    }
    if not args.no_extra:
        extra = {}
        r32 = bench_scan_fwd(max(10, args.steps // 2), 3, dtype=torch.float32)
        a32 = r32["bytes"] / (r32["kernel_ms"] * 1e-3) / 1e9
        extra["selective_scan_fwd_fp32_io"] = {
            "kernel_us": round(r32["kernel_ms"] * 1e3, 2), "GBps": round(a32, 1),
            "frac_hbm": round(a32 / HBM_PEAK_GBPS, 4), "algorithmic_bytes": r32["bytes"]}
        line["extra"] = extra
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline_scan()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
