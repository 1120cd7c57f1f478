#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

Prints ONE JSON line.  A "step" is one pass of the hot path over one batch of synthetic,
seeded input that is already resident in HBM.  Inputs rotate over several buffers whose
total size exceeds the 256 MB Infinity Cache, so every step streams from HBM.

Workloads (``--workload``):
  fp8_gemm   blockwise-FP8 GEMM, M=4096, DeepSeek-V3 gate_up (K=7168 -> N=36864)   [default, headline]
  quant      per-token-group FP8 quantization, M=16384 K=7168 g=128, fp32 row-major scales
  quant_ue8m0  same, column-major packed UE8M0 scales
The default run reports the headline GEMM as ``value`` and carries the quantizer (both
variants) and the other shapes of the named configurations under ``"also"``.

``roofline.achieved`` is algorithmic bytes (or FLOPs) per launch divided by the average
launch duration measured with HIP events on the launch stream; ``cpu_baseline`` times the CPU
oracle on a bounded sample of the same workload on this host.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
FP8_PEAK_TFLOPS = 5000.0    # dense fp8 MFMA (no sparsity)
INT8_PEAK_TOPS = 5000.0

METRIC = "blockwise-FP8 GEMM TFLOPS & %MFMA peak; quant GB/s & %HBM peak (1 GPU)"


def _time_launches(fn, nbuf, steps, warmup):
    """Run fn(i % nbuf) warmup + steps times on the current stream; returns (wall seconds for the
    timed steps, list of per-launch milliseconds from HIP events)."""
    import torch

    for i in range(warmup):
        fn(i % nbuf)
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        evs[i][0].record()
        fn(i % nbuf)
        evs[i][1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, [a.elapsed_time(b) for a, b in evs]


def bench_quant(steps, warmup, ue8m0, with_cpu):
    import torch

    from sglang_amd import fp8_kernel
    from sglang_amd.workloads import make_activation, quant_algorithmic_bytes

    dev = torch.device("cuda:0")
    M, K, G = 16384, 7168, 128
    nbuf = 4
    base = make_activation(M, K, zero_group_frac=1e-4, zero_elem_frac=1e-4)
    xs = [base.to(dev)]
    for i in range(1, nbuf):  # distinct buffers; rolling the rows keeps the distribution and costs no host time
        xs.append(torch.roll(xs[0], shifts=i * 97, dims=0).contiguous())
    qs = [torch.empty(M, K, dtype=torch.float8_e4m3fn, device=dev) for _ in range(nbuf)]
    ss = [fp8_kernel.create_per_token_group_quant_fp8_output_scale((M, K), dev, G, ue8m0, ue8m0, ue8m0)
          for _ in range(nbuf)]
    from sglang_amd.sgl_kernel import sgl_per_token_group_quant_fp8

    def step(i):
        sgl_per_token_group_quant_fp8(xs[i], qs[i], ss[i], G, 1e-10, -448.0, 448.0, ue8m0, enable_v2=ue8m0)

    wall, ms = _time_launches(step, nbuf, steps, warmup)
    alg = quant_algorithmic_bytes(M, K, G, 2, ue8m0)
    avg_ms = sum(ms) / len(ms)
    rec = {
        "workload": ("quant_ue8m0" if ue8m0 else "quant") + f" M={M} K={K} g={G} bf16->e4m3fn "
        + ("col-major packed UE8M0 scales (v2 arithmetic)" if ue8m0 else "row-major fp32 scales (v1 arithmetic)"),
        "value": alg / (wall / steps) / 1e9,
        "unit": "GB/s",
        "ms_per_step": wall / steps * 1e3,
        "kernel_ms_avg": avg_ms,
        "kernel_ms_median": statistics.median(ms),
        "kernel_ms_p20_p80": [sorted(ms)[len(ms) // 5], sorted(ms)[len(ms) * 4 // 5]],
        "dtype": "bf16->fp8(e4m3fn), fp32 arithmetic",
        "roofline": {
            "bound": "hbm", "achieved": alg / (avg_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": alg / (avg_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "algorithmic_bytes": alg,
        },
    }
    if with_cpu:
        from oracle import oracle

        rows = 2048  # 1/8 of the batch
        xs_cpu = base[:rows].contiguous()
        oracle.group_quant(xs_cpu[:64], G, mode="mul" if ue8m0 else "div", layout="ue8m0" if ue8m0 else "row")
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < 10.0:
            oracle.group_quant(xs_cpu, G, mode="mul" if ue8m0 else "div", layout="ue8m0" if ue8m0 else "row",
                               pow2_floor=0.0 if ue8m0 else 1e-10)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        rec["cpu_baseline"] = {
            "value": quant_algorithmic_bytes(rows, K, G, 2, ue8m0) / dt / 1e9, "unit": "GB/s",
            "cores": oracle.num_threads(), "kind": "port",
            "sample": f"first {rows} of {M} rows, {reps} repetitions (~10 s), C oracle with OpenMP",
        }
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="default")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path is measured on ONE GPU; it has no collectives and --gpus N>1 is not run "
              "(see DESIGN.md, 'How the path shards').", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from sglang_amd import _lib

    _lib.lib()  # fail loudly if the HIP library is missing

    with_cpu = not args.no_cpu
    if args.workload in ("quant", "quant_ue8m0"):
        rec = bench_quant(args.steps, args.warmup, args.workload == "quant_ue8m0", with_cpu)
        also = []
    else:
        rec = bench_quant(args.steps, args.warmup, False, with_cpu)
        also = [bench_quant(args.steps, args.warmup, True, False)]

    line = {
        "metric": METRIC,
        "value": rec["value"],
        "unit": rec["unit"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": rec["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": rec["dtype"],
        "data": "synthetic (seeded torch.Generator on CPU, copied to HBM before timing)",
        "config": {"workload": rec["workload"]},
        "roofline": rec["roofline"],
        "kernel_ms": {"avg": rec["kernel_ms_avg"], "median": rec["kernel_ms_median"],
                      "p20_p80": rec["kernel_ms_p20_p80"]},
    }
    if "cpu_baseline" in rec:
        line["cpu_baseline"] = rec["cpu_baseline"]
    if also:
        line["also"] = also
    print(json.dumps(line))


if __name__ == "__main__":
    main()
