#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--quick]

Prints ONE JSON line (kept short: every number has four significant digits).  A "step" is one pass of
the hot path over one batch of seeded synthetic input that is already resident in HBM; weights rotate
over several buffers so that bandwidth-bound steps stream from HBM rather than from the 256 MB
Infinity Cache.

--workload:
  all          (default) headline = blockwise-FP8 GEMM, M=4096, DeepSeek-V3 gate_up K=7168 -> N=36864, as
               `value`; every other configuration the baseline names as short rows under "also"; the
               two quantizer rows (M=16384, K=7168) under "quant", last in the line
  fp8_gemm     the headline alone          quant / quant_ue8m0   one quantizer variant alone
  fp8_decode   FP8 gate_up at M=1          int8_gemm             INT8 gate_up (K=4096 -> N=28672) at M=4096
  fp8:M:K:N    any blockwise-FP8 linear    int8:M:K:N            any INT8 linear
  fp8_ue8m0:M:K:N  the same linear with power-of-two (UE8M0) scales on both operands
  fp8_linear:M:K:N  a whole block-FP8 linear, bf16 in -> bf16 out, one call (fp8_linear2: quantizer call + GEMM call)
  fp8_grouped:E:ROWS:K:N  grouped FP8 GEMM of E experts with ROWS token rows each (mixture-of-experts)
  fp8_ceiling[:M:K:N]  the large-M FP8 kernel with the global loads of its K loop taken out, on the headline's operands
               (what schedule and sustained clock allow once memory is out of the picture; the result is not the product)
  mfma_stream  the kernels' fp8 matrix-instruction streams with all operands in registers, on every CU at once: what the
               chip's power management lets the matrix pipes sustain on the benchmark's operand values (and on zeros)
  copy         a plain 256 MiB device copy (calibration of the HBM traffic counters)
  silu_quant   silu(gate) * up fused in front of the group quantizer (packed UE8M0 scales)
  per_token_fp8 / per_token_int8 / per_tensor_fp8 / block_cast   the other quantizers of the path

Per-launch durations are HIP events on the launch stream (torch's current stream, which is the stream
handed to the C ABI).  `roofline.achieved` = algorithmic FLOPs (2*M*N*K) or bytes per launch / MEDIAN
launch duration, the one basis of every `roofline.frac`; `kernel_ms.b2b` is the average over the same launches
queued back to back between one event pair (no per-launch event overhead; for kernels of tens of microseconds it
also hides the tail of one launch behind the head of the next) and `roofline.frac_b2b` the fraction on it.  `cpu_baseline` times the CPU oracle on a bounded sample of the
same workload on this host's cores.
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

HBM_PEAK_GBS = 8000.0     # MI355X HBM3E
FP8_PEAK_TFLOPS = 5000.0  # dense fp8 MFMA, no sparsity
INT8_PEAK_TOPS = 5000.0   # dense int8 MFMA

METRIC = "blockwise-FP8 GEMM TFLOPS & %MFMA peak; quant GB/s & %HBM peak (1 GPU)"
DATA = ("synthetic, seeded, resident in HBM before the timed region; activations bf16 N(0,1) + 0.1% x50 outliers quantized "
        "1x128 by the GPU quantizer; FP8 weights N(0,0.02) quantized per 128x128 block (drawn on the device); INT8 weights "
        "N(0,0.02) quantized per channel, INT8 activations the same bf16 data quantized per token by the GPU quantizer")


def r4(x):
    """Four significant digits (keeps the JSON line short)."""
    if isinstance(x, float):
        return float(f"{x:.4g}")
    if isinstance(x, dict):
        return {k: r4(v) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [r4(v) for v in x]
    return x


def _time_launches(fn, nbuf, steps, warmup):
    """fn(i % nbuf) is launched warmup + steps times on the current stream.  Returns (wall seconds of the timed
    steps, per-launch milliseconds from HIP events, back-to-back average milliseconds)."""
    import torch

    for i in range(warmup):
        fn(i % nbuf)
    torch.cuda.synchronize()
    # short kernels: keep warming up until ~30 ms of launches have run, so that clocks are up before the timed steps
    t_w = time.perf_counter()
    extra = 0
    while time.perf_counter() - t_w < 0.03 and extra < 2000:
        fn(extra % nbuf)
        extra += 1
        if extra % 32 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        evs[i][0].record()
        fn(i % nbuf)
        evs[i][1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        fn(i % nbuf)
    e1.record()
    torch.cuda.synchronize()
    return wall, [a.elapsed_time(b) for a, b in evs], e0.elapsed_time(e1) / steps


def _stats(ms, b2b):
    s = sorted(ms)
    return {"median": statistics.median(ms), "p20_p80": [s[len(s) // 5], s[len(s) * 4 // 5]], "b2b": b2b}


def _cpu_time_boxed(fn, seconds=10.0):
    fn()  # page in, spin up the OpenMP team
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < seconds:
        fn()
        reps += 1
    return (time.perf_counter() - t0) / reps, reps


def _roofline(flops, nbytes, st, peak_ops, unit_ops):
    """Which roof binds (time at peak MFMA rate vs time at peak HBM rate) and the achieved fraction of it.  ONE basis
    for every row: `achieved` and `frac` use the MEDIAN of the per-launch HIP-event durations.  `frac_b2b` is the same
    fraction on the average over the event-bracketed run of back-to-back launches, printed beside it: for launches of
    tens of microseconds the two event records around each launch cost a visible share of the median, while the
    back-to-back figure hides the tail of one launch behind the head of the next."""
    ms = st["median"]
    if flops / (peak_ops * 1e12) >= nbytes / (HBM_PEAK_GBS * 1e9):
        a = flops / (ms * 1e-3) / 1e12
        return {"bound": "mfma", "achieved": a, "peak": peak_ops, "unit": unit_ops, "frac": a / peak_ops, "traffic": None,
                "per_launch": flops, "basis": "median launch", "frac_b2b": flops / (st["b2b"] * 1e-3) / 1e12 / peak_ops}
    a = nbytes / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": a, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": a / HBM_PEAK_GBS, "traffic": None,
            "per_launch": nbytes, "basis": "median launch", "frac_b2b": nbytes / (st["b2b"] * 1e-3) / 1e9 / HBM_PEAK_GBS}


# ------------------------------------------------------------------------------------------ quantizer

def bench_quant(steps, warmup, ue8m0, with_cpu):
    import torch

    from sglang_amd import _lib, fp8_kernel
    from sglang_amd.sgl_kernel import sgl_per_token_group_quant_fp8
    from sglang_amd.workloads import make_activation, quant_algorithmic_bytes

    dev = torch.device("cuda:0")
    M, K, G = 16384, 7168, 128
    nbuf = 4
    base = make_activation(M, K, zero_group_frac=1e-4, zero_elem_frac=1e-4)
    xs = [base.to(dev)]
    for i in range(1, nbuf):  # distinct buffers; rolling the rows keeps the distribution
        xs.append(torch.roll(xs[0], shifts=i * 97, dims=0).contiguous())
    qs = [torch.empty(M, K, dtype=torch.float8_e4m3fn, device=dev) for _ in range(nbuf)]
    ss = [fp8_kernel.create_per_token_group_quant_fp8_output_scale((M, K), dev, G, ue8m0, ue8m0, ue8m0)
          for _ in range(nbuf)]

    # one check through the reference-named entry point, then the timed loop calls the C ABI directly with the same
    # arguments: a 60 us kernel must not be timed together with the Python operator dispatch
    sgl_per_token_group_quant_fp8(xs[0], qs[0], ss[0], G, 1e-10, -448.0, 448.0, ue8m0, enable_v2=ue8m0)
    L = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    if ue8m0:  # v2 arithmetic (q = x * 448/amax), packed exponents, words column-major
        tail = (_lib.QUANT_MUL, _lib.SCALE_UE8M0_PACKED, 0.0, 1, ss[0].stride(1))
    else:      # v1 arithmetic (q = x / s), fp32 scales row-major
        tail = (_lib.QUANT_DIV, _lib.SCALE_F32, 1e-10, K // G, 1)
    args = [(xs[i].data_ptr(), _lib.BF16, qs[i].data_ptr(), _lib.FP8_E4M3FN, ss[i].data_ptr(), M, K, G, 1e-10, -448.0, 448.0,
             *tail, stream) for i in range(nbuf)]

    def step(i):
        _lib.check(L.mi355_group_quant_8bit(*args[i]))

    wall, ms, b2b = _time_launches(step, nbuf, steps, warmup)
    alg = quant_algorithmic_bytes(M, K, G, 2, ue8m0)
    st = _stats(ms, b2b)
    rec = {
        "workload": f"group quant M={M} K={K} g={G} bf16->e4m3fn, "
        + ("column-major packed UE8M0 scales (q = x*448/amax)" if ue8m0 else "row-major fp32 scales (q = x/s)"),
        "value": alg / (wall / steps) / 1e9, "unit": "GB/s", "ms_per_step": wall / steps * 1e3, "kernel_ms": st,
        "dtype": "f32 on bf16 in, e4m3fn out",
        "roofline": _roofline(0, alg, st, FP8_PEAK_TFLOPS, "TFLOP/s"),
    }
    if with_cpu:
        from oracle import oracle

        rows = 2048
        xc = base[:rows].contiguous()
        kw = dict(mode="mul" if ue8m0 else "div", layout="ue8m0" if ue8m0 else "row", pow2_floor=0.0 if ue8m0 else 1e-10)
        dt, reps = _cpu_time_boxed(lambda: oracle.group_quant(xc, G, **kw))
        rec["cpu_baseline"] = {
            "value": quant_algorithmic_bytes(rows, K, G, 2, ue8m0) / dt / 1e9, "unit": "GB/s",
            "cores": oracle.num_threads(), "kind": "port",
            "sample": f"first {rows} of {M} rows, {reps} reps in ~10 s, C oracle with OpenMP",
        }
    return rec


# ------------------------------------------------------------------------------------------ FP8 GEMM

def device_block_fp8_weight(N, K, gen, dev):
    """N(0, 0.02) weights quantized per 128x128 block on the device (same arithmetic as workloads.block_cast_to_fp8):
    (e4m3fn [N, K], fp32 scales [ceil(N/128), ceil(K/128)]).  Rows are drawn in slabs to bound the fp32 scratch."""
    import torch

    from sglang_amd.workloads import cdiv

    Kp = cdiv(K, 128) * 128
    q = torch.empty(N, K, dtype=torch.float8_e4m3fn, device=dev)
    s = torch.empty(cdiv(N, 128), cdiv(K, 128), dtype=torch.float32, device=dev)
    slab = 128 * 32
    for n0 in range(0, N, slab):
        n1 = min(N, n0 + slab)
        rows = cdiv(n1 - n0, 128) * 128
        w = torch.zeros(rows, Kp, dtype=torch.float32, device=dev)
        w[: n1 - n0, :K] = torch.randn(n1 - n0, K, generator=gen, device=dev) * 0.02
        v = w.view(rows // 128, 128, Kp // 128, 128)
        amax = v.abs().amax(dim=(1, 3), keepdim=True).clamp(min=1e-4)
        q[n0:n1] = (v * (448.0 / amax)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(rows, Kp)[: n1 - n0, :K]
        s[n0 // 128: n0 // 128 + rows // 128] = (amax / 448.0).view(rows // 128, Kp // 128)
    return q, s


def bench_fp8_gemm(name, M, K, N, steps, warmup, with_cpu, w8a16_cpu=False):
    """One blockwise-FP8 linear through sgl_kernel.fp8_blockwise_scaled_mm (or, for N or K not a multiple of 128,
    through w8a8_block_fp8_matmul)."""
    import torch

    from sglang_amd import _lib, fp8_kernel, sgl_kernel
    from sglang_amd.workloads import cdiv, fp8_gemm_algorithmic_bytes, gemm_flops, make_activation

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(N * 10007 + K)
    nbuf = max(2, min(6, int(600e6 // (N * K)) + 1))  # rotate through > 512 MB of weights when they are small
    ws, wss = zip(*[device_block_fp8_weight(N, K, gen, dev) for _ in range(nbuf)])
    x = make_activation(M, K).to(dev)
    aligned = N % 128 == 0 and K % 128 == 0
    x_q, x_s = fp8_kernel.per_token_group_quant_fp8(x, 128, column_major_scales=aligned)

    if aligned:
        def step(i):
            return sgl_kernel.fp8_blockwise_scaled_mm(x_q, ws[i].t(), x_s, wss[i].t(), torch.bfloat16)
    else:
        def step(i):
            return fp8_kernel.w8a8_block_fp8_matmul(x_q, ws[i], x_s, wss[i], [128, 128], torch.bfloat16)

    direct = M <= 256 or N * K <= 16e6  # launches of tens of microseconds
    if direct:
        # decode-sized steps take tens of microseconds: call the C ABI directly with preallocated output and workspace,
        # so that the host keeps the queue full and the events time kernels rather than Python
        L = _lib.lib()
        wsb = L.mi355_fp8_blockwise_mm_workspace_bytes(M, N, K)
        wsbuf = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)
        outs = [torch.empty(M, N, dtype=torch.bfloat16, device=dev) for _ in range(nbuf)]
        stream = torch.cuda.current_stream().cuda_stream
        args = [(x_q.data_ptr(), ws[i].data_ptr(), x_s.data_ptr(), wss[i].data_ptr(), outs[i].data_ptr(), _lib.BF16, M, N, K,
                 x_q.stride(0), ws[i].stride(0), x_s.stride(0), x_s.stride(1), wss[i].stride(0), wss[i].stride(1),
                 outs[i].stride(0), wsbuf.data_ptr(), wsb, stream) for i in range(nbuf)]

        def step(i):  # noqa: F811
            _lib.check(L.mi355_fp8_blockwise_mm(*args[i]))

    wall, ms, b2b = _time_launches(step, nbuf, steps, warmup)
    st = _stats(ms, b2b)
    flops, nbytes = gemm_flops(M, N, K), fp8_gemm_algorithmic_bytes(M, N, K)
    plan = _lib.gemm_plan("fp8", M, N, K, aligned=(K % 16 == 0))
    rec = {
        "workload": f"fp8_gemm {name} M={M} K={K} N={N} (e4m3fn x e4m3fn, 1x128 / 128x128 fp32 scales, bf16 out"
        + (", direct C-ABI calls)" if direct else ")"),
        "value": flops / (wall / steps) / 1e12, "unit": "TFLOP/s", "ms_per_step": wall / steps * 1e3, "kernel_ms": st,
        "dtype": "fp8(e4m3fn) MFMA, f32 accumulate", "kernel": plan["kernel"] + (f" x{plan['splits']}" if plan["splits"] > 1 else ""),
        "roofline": _roofline(flops, nbytes, st, FP8_PEAK_TFLOPS, "TFLOP/s"),
    }
    if with_cpu:
        from oracle import oracle

        ms_, ns_ = min(M, 64), min(N, 1024)
        a_c, sa_c = x_q[:ms_].cpu().contiguous(), x_s[:ms_].cpu().contiguous()
        w_c, sw_c = ws[0][:ns_].cpu().contiguous(), wss[0][: cdiv(ns_, 128)].cpu().contiguous()
        dt, reps = _cpu_time_boxed(lambda: oracle.fp8_blockwise_mm(a_c, w_c, sa_c, sw_c, torch.bfloat16))
        rec["cpu_baseline"] = {
            "value": gemm_flops(ms_, ns_, K) / dt / 1e12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{ms_} tokens x {ns_} channels x K={K}, {reps} reps in ~10 s, C oracle with OpenMP (fp64 block sums)",
        }
        # the reference's torch-native formulation (test_block_fp8.py:273-325) on the same sample, fp32 matmul per K block
        A32, B32 = a_c.float(), w_c.float()

        def native():
            C = torch.zeros(ms_, ns_)
            for kb in range(cdiv(K, 128)):
                ks = slice(kb * 128, min((kb + 1) * 128, K))
                C.add_((A32[:, ks] @ B32[:, ks].T) * (sa_c[:, kb:kb + 1] * sw_c[:, kb].repeat_interleave(128)[None, :ns_]))
            return C.to(torch.bfloat16)

        dt2, reps2 = _cpu_time_boxed(native, 5.0)
        rec["cpu_torch_native"] = {"value": gemm_flops(ms_, ns_, K) / dt2 / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
                                   "kind": "port", "sample": f"same sample, {reps2} reps in ~5 s, torch fp32 matmul per K block"}
        if w8a16_cpu:
            # the arithmetic of the reference's own CPU kernel (sgl-kernel/csrc/cpu/gemm_fp8.cpp:471-551): bf16 activations are
            # NOT quantized, the fp8 weight is dequantized per block and multiplied in bf16 (w8a16) - a different operator
            xb = x[:ms_].cpu()
            wdq = (B32 * sw_c.repeat_interleave(128, 0)[:ns_].repeat_interleave(128, 1)[:, :K]).to(torch.bfloat16)
            dt3, reps3 = _cpu_time_boxed(lambda: xb @ wdq.T, 5.0)
            rec["cpu_w8a16_shape"] = {"value": gemm_flops(ms_, ns_, K) / dt3 / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
                                      "kind": "port", "sample": f"same sample, {reps3} reps in ~5 s, bf16 x dequantized-weight matmul "
                                      "(w8a16: what the reference's CPU build computes; different arithmetic, weight dequantized once)"}
    return rec


# ------------------------------------------------------------------------------------------ INT8 GEMM

def bench_fp8_ue8m0_gemm(name, M, K, N, steps, warmup):
    """Blockwise-FP8 linear with power-of-two (UE8M0) scales on both operands: the weight re-quantized by
    requant_weight_ue8m0, the activation quantized with packed exponents; N and K multiples of 128."""
    import torch

    from sglang_amd import _lib, fp8_kernel, fp8_utils, ops
    from sglang_amd.workloads import fp8_gemm_algorithmic_bytes, gemm_flops, make_activation

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(N * 10007 + K)
    nbuf = max(2, min(6, int(600e6 // (N * K)) + 1))
    ws, wss = [], []
    for _ in range(nbuf):
        w_q, w_s = device_block_fp8_weight(N, K, gen, dev)
        w2, sw = fp8_utils.requant_weight_ue8m0(w_q, w_s, [128, 128])
        ws.append(w2)
        wss.append(sw)
    x = make_activation(M, K).to(dev)
    x_q, x_s = fp8_kernel.sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True, scale_tma_aligned=True,
                                                           scale_ue8m0=True, enable_v2=True)

    def step(i):
        return ops.fp8_blockwise_mm_ue8m0(x_q, ws[i], x_s, wss[i], torch.bfloat16)

    if M <= 256 or N * K <= 16e6:
        L = _lib.lib()
        wsb = L.mi355_fp8_blockwise_mm_ue8m0_workspace_bytes(M, N, K)
        wsbuf = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)
        outs = [torch.empty(M, N, dtype=torch.bfloat16, device=dev) for _ in range(nbuf)]
        stream = torch.cuda.current_stream().cuda_stream
        args = [(x_q.data_ptr(), ws[i].data_ptr(), x_s.data_ptr(), wss[i].data_ptr(), None, outs[i].data_ptr(), _lib.BF16, M, N, K,
                 x_q.stride(0), ws[i].stride(0), x_s.stride(1), wss[i].stride(0), wss[i].stride(1), outs[i].stride(0),
                 wsbuf.data_ptr(), wsb, stream) for i in range(nbuf)]

        def step(i):  # noqa: F811
            _lib.check(L.mi355_fp8_blockwise_mm_ue8m0(*args[i]))

    wall, ms, b2b = _time_launches(step, nbuf, steps, warmup)
    st = _stats(ms, b2b)
    flops, nbytes = gemm_flops(M, N, K), fp8_gemm_algorithmic_bytes(M, N, K)
    plan = _lib.gemm_plan("fp8", M, N, K)
    # kernels whose MFMA applies the exponents
    hw = plan["kernel"] in ("pingpong", "dma3", "decode", "decode_wavesplit") and K % 128 == 0
    kern = plan["kernel"] + (" (MFMA-applied scales)" if hw else " after unpack")
    return {
        "workload": f"fp8_gemm_ue8m0 {name} M={M} K={K} N={N} (e4m3fn x e4m3fn, packed UE8M0 scales on both sides, bf16 out)",
        "value": flops / (wall / steps) / 1e12, "unit": "TFLOP/s", "ms_per_step": wall / steps * 1e3, "kernel_ms": st,
        "dtype": "fp8(e4m3fn) MFMA with block scales, f32 accumulate", "kernel": kern,
        "roofline": _roofline(flops, nbytes, st, FP8_PEAK_TFLOPS, "TFLOP/s"),
    }


def bench_fp8_grouped_gemm(E, m_per, K, N, steps, warmup):
    """Grouped blockwise-FP8 GEMM (the expert GEMMs of a mixture-of-experts layer): E experts with m_per stacked token
    rows each, one [N, K] weight per expert; the shapes of sgl-kernel/benchmark/bench_fp8_blockwise_group_gemm.py.  One
    step is the whole call: schedule kernel, scale re-layout and the GEMM."""
    import torch

    from sglang_amd import _lib, fp8_kernel
    from sglang_amd.workloads import make_activation

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(N * 10007 + K + E)
    T = E * m_per
    nbuf = max(2, min(6, int(600e6 // (E * N * K)) + 1))
    ws, wss = [], []
    for _ in range(nbuf):
        w_q, w_s = device_block_fp8_weight(E * N, K, gen, dev)
        ws.append(w_q.view(E, N, K))
        wss.append(w_s.view(E, N // 128, K // 128))
    x = make_activation(T, K).to(dev)
    x_q, x_s = fp8_kernel.sglang_per_token_group_quant_fp8(x, 128)
    sizes = torch.tensor([[m_per, N, K]] * E, dtype=torch.int32, device=dev)
    offsets = torch.arange(E, dtype=torch.int32, device=dev) * m_per
    L = _lib.lib()
    wsb = L.mi355_fp8_blockwise_scaled_grouped_mm_workspace_bytes(E, T, N, K)
    wsbuf = torch.empty(wsb, dtype=torch.uint8, device=dev)
    outs = [torch.empty(T, N, dtype=torch.bfloat16, device=dev) for _ in range(nbuf)]
    stream = torch.cuda.current_stream().cuda_stream
    args = [(x_q.data_ptr(), ws[i].data_ptr(), x_s.data_ptr(), wss[i].data_ptr(), outs[i].data_ptr(), _lib.BF16, sizes.data_ptr(),
             offsets.data_ptr(), E, T, N, K, x_q.stride(0), K, N * K, x_s.stride(0), x_s.stride(1), wss[i].stride(0),
             wss[i].stride(1), wss[i].stride(2), N, wsbuf.data_ptr(), wsb, stream) for i in range(nbuf)]

    def step(i):
        _lib.check(L.mi355_fp8_blockwise_scaled_grouped_mm(*args[i]))

    wall, ms, b2b = _time_launches(step, nbuf, steps, warmup)
    st = _stats(ms, b2b)
    kb = K // 128
    flops = 2.0 * T * N * K
    nbytes = float(E * N * K + T * K + 4 * T * kb + 4 * E * (N // 128) * kb + 2 * T * N)
    plan = _lib.grouped_gemm_plan(E, T, N, K)
    return {
        "workload": f"fp8_grouped_gemm E={E} rows/expert={m_per} K={K} N={N} (e4m3fn x e4m3fn, 1x128 / 128x128 fp32 scales, bf16 out)",
        "value": flops / (wall / steps) / 1e12, "unit": "TFLOP/s", "ms_per_step": wall / steps * 1e3, "kernel_ms": st,
        "dtype": "fp8(e4m3fn) MFMA, f32 accumulate", "kernel": f"{plan['kernel']} {plan['small_tile']} (+ schedule, scale re-layout)",
        "roofline": _roofline(flops, nbytes, st, FP8_PEAK_TFLOPS, "TFLOP/s"),
    }


def bench_fp8_ceiling(M, K, N, steps, warmup):
    """The large-M FP8 kernel with the global loads of its K loop taken out (mi355_fp8_blockwise_mm_kloop_ceiling), on the
    operands of bench_fp8_gemm.  `value` is what the matrix instructions, promotion FMAs, LDS reads, barriers and epilogue
    of the operator sustain on these operand values when nothing is fetched inside the loop; the operator itself is timed
    in the same call on the same buffers ("operator_ms")."""
    import torch

    from sglang_amd import _lib, fp8_kernel
    from sglang_amd.workloads import fp8_gemm_algorithmic_bytes, gemm_flops, make_activation

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(N * 10007 + K)
    nbuf = 2
    ws, wss = zip(*[device_block_fp8_weight(N, K, gen, dev) for _ in range(nbuf)])
    x = make_activation(M, K).to(dev)
    x_q, x_s = fp8_kernel.per_token_group_quant_fp8(x, 128, column_major_scales=True)
    L = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    outs = [torch.empty(M, N, dtype=torch.bfloat16, device=dev) for _ in range(nbuf)]
    wsb = L.mi355_fp8_blockwise_mm_workspace_bytes(M, N, K)
    wsbuf = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)
    common = [(x_q.data_ptr(), ws[i].data_ptr(), x_s.data_ptr(), wss[i].data_ptr(), outs[i].data_ptr(), _lib.BF16, M, N, K,
               x_q.stride(0), ws[i].stride(0), x_s.stride(0), x_s.stride(1), wss[i].stride(0), wss[i].stride(1),
               outs[i].stride(0)) for i in range(nbuf)]

    def operator(i):
        _lib.check(L.mi355_fp8_blockwise_mm(*common[i], wsbuf.data_ptr(), wsb, stream))

    def ceiling(i):
        _lib.check(L.mi355_fp8_blockwise_mm_kloop_ceiling(*common[i], stream))

    _, ms_op, b2b_op = _time_launches(operator, nbuf, steps, warmup)
    wall, ms, b2b = _time_launches(ceiling, nbuf, steps, warmup)
    st, st_op = _stats(ms, b2b), _stats(ms_op, b2b_op)
    flops, nbytes = gemm_flops(M, N, K), fp8_gemm_algorithmic_bytes(M, N, K)
    return {
        "workload": f"fp8_ceiling M={M} K={K} N={N} (the large-M FP8 kernel without the global loads of its K loop; not the product)",
        "value": flops / (wall / steps) / 1e12, "unit": "TFLOP/s", "ms_per_step": wall / steps * 1e3, "kernel_ms": st,
        "dtype": "fp8(e4m3fn) MFMA, f32 accumulate", "kernel": "pingpong, K-loop loads removed",
        "roofline": _roofline(flops, nbytes, st, FP8_PEAK_TFLOPS, "TFLOP/s"),
        "operator_ms": st_op, "operator_frac": flops / (st_op["median"] * 1e-3) / 1e12 / FP8_PEAK_TFLOPS,
    }


def bench_mfma_stream(steps, warmup):
    """The fp8 matrix-instruction streams of the large-M kernels with every operand in registers (mi355_probe_fp8_mfma_stream),
    256 workgroups of 8 waves: fp32-scale stream (C = 0 + four promotion FMAs), in-place stream, MFMA only; each on operand
    values distributed like the benchmark's (quantized N(0,1) activations x block-quantized N(0, 0.02) weights) and on zeros."""
    import torch

    from sglang_amd import _lib, fp8_kernel

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(11)
    n = 8 * 4 * 64 * 32
    x = torch.randn(n // 128, 128, generator=gen, device=dev).to(torch.bfloat16)
    a_real, _ = fp8_kernel.per_token_group_quant_fp8(x, 128)
    w_q, _ = device_block_fp8_weight(n // 128, 128, gen, dev)
    zeros = torch.zeros(n, dtype=torch.uint8, device=dev)
    out = torch.empty(256 * 512, dtype=torch.float32, device=dev)
    L = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    iters = 2000
    flops = 256.0 * 8 * iters * 16 * 2 * 16 * 16 * 128
    # INT8 operands as bench_int8_gemm has them: per-token quantized N(0,1) activations, per-channel quantized N(0, 0.02) weights
    xi = torch.randn(n // 4096, 4096, generator=gen, device=dev)
    a_i8 = torch.round(xi * (127.0 / xi.abs().amax(dim=1, keepdim=True))).to(torch.int8)
    wi = torch.randn(n // 4096, 4096, generator=gen, device=dev) * 0.02
    w_i8 = torch.round(wi * (127.0 / wi.abs().amax(dim=1, keepdim=True))).to(torch.int8)
    out_i = torch.empty(256 * 512, dtype=torch.int32, device=dev)
    rows = []
    for data, (pa, pb), (qa, qb) in (("benchmark operand values", (a_real, w_q), (a_i8, w_i8)), ("zeros", (zeros, zeros), (zeros, zeros))):
        for mode, name in ((0, "C=0 + 4 promotion FMAs per MFMA (fp32-scale kernel)"), (1, "accumulate in place (UE8M0 kernel)"),
                           (2, "MFMA only"), (3, "MFMA only, 32x32x64 instead of 16x16x128 (not used)"),
                           (10, "int8 16x16x64 in place (INT8 kernels)"), (11, "int8 32x32x32 in place (not used)")):
            def step(i, mode=mode, pa=pa, pb=pb, qa=qa, qb=qb):
                if mode >= 10:
                    _lib.check(L.mi355_probe_int8_mfma_stream(mode - 10, 256, iters, qa.data_ptr(), qb.data_ptr(), out_i.data_ptr(), stream))
                else:
                    _lib.check(L.mi355_probe_fp8_mfma_stream(mode, 256, iters, pa.data_ptr(), pb.data_ptr(), out.data_ptr(), stream))

            wall, ms, b2b = _time_launches(step, 1, max(10, steps // 2), 3)
            st = _stats(ms, b2b)
            tf = flops / (st["median"] * 1e-3) / 1e12
            rows.append({"stream": name, "operands": data, "ms": st["median"], "TFLOP/s": tf, "frac": tf / FP8_PEAK_TFLOPS,
                         # two waves per SIMD issue 32-cycle instructions back to back: the clock at which the time fits
                         "clock_GHz_if_pipe_full": 2.0 * iters * 16 * 32 / (st["median"] * 1e-3) / 1e9})
    head = rows[0]
    st = {"median": head["ms"], "p20_p80": [head["ms"], head["ms"]], "b2b": head["ms"]}
    return {
        "workload": "mfma_stream (fp8 16x16x128 matrix instructions, operands in registers, 256 workgroups x 8 waves; not a GEMM)",
        "value": head["TFLOP/s"], "unit": "TFLOP/s", "ms_per_step": head["ms"], "kernel_ms": st,
        "dtype": "fp8(e4m3fn) MFMA, f32 accumulate", "kernel": "mfma_stream",
        "roofline": _roofline(flops, 0.0, st, FP8_PEAK_TFLOPS, "TFLOP/s"), "streams": rows,
    }


def bench_fp8_linear(M, K, N, steps, warmup, two_step):
    """A whole block-FP8 linear from bf16 activations to bf16 output: the one-call entry point (at decode sizes the GEMM
    kernel quantizes in its prologue), or, with two_step, quantizer call + GEMM call as the reference's wrappers do."""
    import torch

    from sglang_amd import _lib
    from sglang_amd.workloads import fp8_gemm_algorithmic_bytes, gemm_flops, make_activation

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(N * 10007 + K)
    nbuf = max(2, min(6, int(600e6 // (N * K)) + 1))
    ws = [device_block_fp8_weight(N, K, gen, dev) for _ in range(nbuf)]
    x = make_activation(M, K).to(dev)
    L = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    outs = [torch.empty(M, N, dtype=torch.bfloat16, device=dev) for _ in range(nbuf)]
    kb = K // 128
    if two_step:
        q = torch.empty(M, K, dtype=torch.float8_e4m3fn, device=dev)
        pitch = (M + 3) // 4 * 4
        sa = torch.empty(kb, pitch, dtype=torch.float32, device=dev)
        wsb = L.mi355_fp8_blockwise_mm_workspace_bytes(M, N, K)
        wsbuf = torch.empty(max(wsb, 256), dtype=torch.uint8, device=dev)

        def step(i):
            _lib.check(L.mi355_group_quant_8bit(x.data_ptr(), _lib.BF16, q.data_ptr(), _lib.FP8_E4M3FN, sa.data_ptr(), M, K, 128, 1e-10,
                                                -448.0, 448.0, _lib.QUANT_DIV, _lib.SCALE_F32, 0.0, 1, pitch, stream))
            _lib.check(L.mi355_fp8_blockwise_mm(q.data_ptr(), ws[i][0].data_ptr(), sa.data_ptr(), ws[i][1].data_ptr(), outs[i].data_ptr(),
                                                _lib.BF16, M, N, K, K, K, 1, pitch, ws[i][1].stride(0), ws[i][1].stride(1), N,
                                                wsbuf.data_ptr(), wsb, stream))
    else:
        wsb = L.mi355_fp8_block_linear_workspace_bytes(M, N, K)
        wsbuf = torch.empty(max(wsb, 256), dtype=torch.uint8, device=dev)

        def step(i):
            _lib.check(L.mi355_fp8_block_linear(x.data_ptr(), _lib.BF16, ws[i][0].data_ptr(), ws[i][1].data_ptr(), ws[i][1].stride(0),
                                                ws[i][1].stride(1), None, outs[i].data_ptr(), _lib.BF16, M, N, K, K, N,
                                                wsbuf.data_ptr(), wsb, stream))

    wall, ms, b2b = _time_launches(step, nbuf, steps, warmup)
    st = _stats(ms, b2b)
    flops, nbytes = gemm_flops(M, N, K), fp8_gemm_algorithmic_bytes(M, N, K) + M * K
    plan = _lib.gemm_plan("fp8", M, N, K) if two_step else _lib.block_linear_plan(M, N, K)
    label = ("quantizer + " if two_step or plan["quantizer"] == "launch" else "") + plan["kernel"] + ("" if two_step or plan["quantizer"] == "launch" else " (quantizer in its prologue)")
    return {
        "workload": f"fp8_linear{'_two_step' if two_step else ''} M={M} K={K} N={N} (bf16 in, 1x128 quantization, blockwise GEMM, bf16 out)",
        "value": flops / (wall / steps) / 1e12, "unit": "TFLOP/s", "ms_per_step": wall / steps * 1e3, "kernel_ms": st,
        "dtype": "fp8(e4m3fn) MFMA, f32 accumulate", "kernel": label,
        "roofline": _roofline(flops, nbytes, st, FP8_PEAK_TFLOPS, "TFLOP/s"),
    }


def bench_int8_gemm(name, M, K, N, steps, warmup, with_cpu=False):
    import torch

    from sglang_amd import _lib, sgl_kernel
    from sglang_amd.workloads import gemm_flops, int8_gemm_algorithmic_bytes

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(N * 10009 + K)
    nbuf = max(2, min(6, int(600e6 // (N * K)) + 1))
    # operands as a W8A8 checkpoint and its activations have them: N(0, 0.02) weights quantized symmetrically per output
    # channel, bf16 N(0, 1) activations (with outliers) quantized per token by the GPU quantizer.  Timing depends on the
    # data through the chip's power state; uniformly random bytes would be the worst case, not a representative one.
    from sglang_amd.int8_kernel import per_token_quant_int8
    from sglang_amd.workloads import make_activation

    ws, sbs = [], []
    for _ in range(nbuf):
        q = torch.empty(N, K, dtype=torch.int8, device=dev)
        sc = torch.empty(N, dtype=torch.float32, device=dev)
        for n0 in range(0, N, 4096):
            w = torch.randn(min(4096, N - n0), K, generator=gen, device=dev) * 0.02
            amax = w.abs().amax(dim=1, keepdim=True).clamp(min=1e-8)
            q[n0:n0 + w.shape[0]] = torch.round(w * (127.0 / amax)).to(torch.int8)
            sc[n0:n0 + w.shape[0]] = (amax / 127.0).view(-1)
        ws.append(q)
        sbs.append(sc)
    sb = sbs[0]
    a, sa = per_token_quant_int8(make_activation(M, K).to(dev))
    bias = torch.randn(N, device=dev, generator=gen).to(torch.bfloat16)

    def step(i):
        return sgl_kernel.int8_scaled_mm(a, ws[i].t(), sa, sbs[i], torch.bfloat16, bias)

    direct = M <= 256 or N * K <= 16e6  # launches of tens of microseconds
    if direct:
        L = _lib.lib()
        wsb = L.mi355_int8_scaled_mm_workspace_bytes(M, N, K)
        wsbuf = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)
        outs = [torch.empty(M, N, dtype=torch.bfloat16, device=dev) for _ in range(nbuf)]
        stream = torch.cuda.current_stream().cuda_stream
        args = [(a.data_ptr(), ws[i].data_ptr(), sa.data_ptr(), sbs[i].data_ptr(), bias.data_ptr(), outs[i].data_ptr(), _lib.BF16,
                 M, N, K, a.stride(0), ws[i].stride(0), outs[i].stride(0), wsbuf.data_ptr(), wsb, stream) for i in range(nbuf)]

        def step(i):  # noqa: F811
            _lib.check(L.mi355_int8_scaled_mm(*args[i]))

    wall, ms, b2b = _time_launches(step, nbuf, steps, warmup)
    st = _stats(ms, b2b)
    ops_, nbytes = gemm_flops(M, N, K), int8_gemm_algorithmic_bytes(M, N, K)
    plan = _lib.gemm_plan("int8", M, N, K)
    rec = {
        "workload": f"int8_gemm {name} M={M} K={K} N={N} (int8 x int8 -> int32, per-token x per-channel scales, bias, bf16 out"
        + (", direct C-ABI calls)" if direct else ")"),
        "value": ops_ / (wall / steps) / 1e12, "unit": "TOP/s", "ms_per_step": wall / steps * 1e3, "kernel_ms": st,
        "dtype": "int8 MFMA, int32 accumulate", "kernel": plan["kernel"] + (f" x{plan['splits']}" if plan["splits"] > 1 else ""),
        "roofline": _roofline(ops_, nbytes, st, INT8_PEAK_TOPS, "TOP/s"),
    }
    if with_cpu:
        from oracle import oracle

        ms_, ns_ = min(M, 64), min(N, 1024)
        a_c, w_c = a[:ms_].cpu().contiguous(), ws[0][:ns_].cpu().contiguous()
        sa_c, sb_c, b_c = sa[:ms_].cpu().view(-1).contiguous(), sb[:ns_].cpu().contiguous(), bias[:ns_].cpu().contiguous()
        dt, reps = _cpu_time_boxed(lambda: oracle.int8_scaled_mm(a_c, w_c, sa_c, sb_c, torch.bfloat16, b_c))
        rec["cpu_baseline"] = {
            "value": gemm_flops(ms_, ns_, K) / dt / 1e12, "unit": "TOP/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{ms_} tokens x {ns_} channels x K={K}, {reps} reps in ~10 s, C oracle with OpenMP (exact int32 matmul + epilogue)",
        }
    return rec


def bench_silu_quant(steps, warmup):
    """silu(gate) * up fused in front of the group quantizer (packed UE8M0 scales), [32768, 2 x 2048] bf16."""
    import torch

    from sglang_amd import _lib, fp8_kernel

    dev = torch.device("cuda:0")
    T, H = 32768, 2048
    nbuf = 3
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    xs = [torch.randn(T, 2 * H, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(nbuf)]
    qs = [torch.empty(T, H, dtype=torch.float8_e4m3fn, device=dev) for _ in range(nbuf)]
    ss = [fp8_kernel.create_per_token_group_quant_fp8_output_scale((T, H), dev, 128, True, True, True) for _ in range(nbuf)]
    L = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    args = [(xs[i].data_ptr(), _lib.BF16, qs[i].data_ptr(), ss[i].data_ptr(), 1, T, H, None, 0, ss[i].stride(1), stream)
            for i in range(nbuf)]

    def step(i):
        _lib.check(L.mi355_silu_mul_group_quant_fp8(*args[i]))

    wall, ms, b2b = _time_launches(step, nbuf, steps, warmup)
    st = _stats(ms, b2b)
    alg = T * H * (4 + 1) + T * (H // 128)
    return {
        "workload": f"silu_mul_quant M={T} H={H} g=128 bf16 [M,2H] -> e4m3fn [M,H], packed UE8M0 scales",
        "value": alg / (wall / steps) / 1e9, "unit": "GB/s", "ms_per_step": wall / steps * 1e3, "kernel_ms": st,
        "dtype": "f32 arithmetic, e4m3fn out", "kernel": "silu_mul_quant", "traffic_key": "silu_mul_quant",
        "roofline": _roofline(0, alg, st, FP8_PEAK_TFLOPS, "TFLOP/s"),
    }


def bench_row_quant(kind, steps, warmup):
    """The other activation / weight quantizers of the path on bf16 data, as HBM-bound kernels: per-token FP8 and INT8
    (one scale per row), per-tensor FP8 (dynamic: absmax pass + quantize pass, the scale word cleared by a fill kernel in
    between) and the 128 x 128 block cast of a weight to power-of-two scales.  Algorithmic bytes: every input element read
    once (twice for the two-pass per-tensor quantizer), every code written once, plus the scales."""
    import torch

    from sglang_amd import _lib

    dev = torch.device("cuda:0")
    L = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator(device=dev)
    gen.manual_seed(9)
    nbuf = 3
    if kind == "block_cast":
        R, C = 36864, 7168
        xs = [(torch.randn(R, C, generator=gen, device=dev, dtype=torch.float32) * 0.02).to(torch.bfloat16) for _ in range(nbuf)]
        qs = [torch.empty(R, C, dtype=torch.float8_e4m3fn, device=dev) for _ in range(nbuf)]
        ss = [torch.empty(R // 128, C // 128, dtype=torch.float32, device=dev) for _ in range(nbuf)]
        step = lambda i: _lib.check(L.mi355_block_cast_to_fp8(xs[i].data_ptr(), _lib.BF16, qs[i].data_ptr(), ss[i].data_ptr(), R, C, stream))
        alg, name, kern = R * C * 3 + 4 * ss[0].numel(), f"block_cast_to_fp8 weight [{R}, {C}] bf16 -> e4m3fn, 128x128 power-of-two scales", "block_cast"
    else:
        from sglang_amd.workloads import make_activation

        M, K = (16384, 4096) if kind == "per_token_int8" else (16384, 7168)
        base = make_activation(M, K).to(dev)
        xs = [base.clone() for _ in range(nbuf)]
        qs = [torch.empty(M, K, dtype=torch.int8 if kind == "per_token_int8" else torch.float8_e4m3fn, device=dev) for _ in range(nbuf)]
        if kind == "per_tensor_fp8":
            ss = [torch.zeros(1, dtype=torch.float32, device=dev) for _ in range(nbuf)]

            def step(i):
                ss[i].zero_()  # the dynamic quantizer merges block maxima into the scale word: it starts from zero
                _lib.check(L.mi355_per_tensor_quant_fp8(xs[i].data_ptr(), _lib.BF16, qs[i].data_ptr(), ss[i].data_ptr(), M * K, 0, None, 0, stream))
            alg, kern = M * K * (2 + 2 + 1) + 4, "per_tensor_absmax + per_tensor_quant"
        else:
            ss = [torch.empty(M, 1, dtype=torch.float32, device=dev) for _ in range(nbuf)]
            fn = L.mi355_per_token_quant_int8 if kind == "per_token_int8" else L.mi355_per_token_quant_fp8
            step = lambda i: _lib.check(fn(xs[i].data_ptr(), _lib.BF16, qs[i].data_ptr(), ss[i].data_ptr(), M, K, stream))
            alg, kern = M * K * 3 + 4 * M, "per_token_quant"
        name = f"{kind}_quant M={M} K={K} bf16"
    wall, ms, b2b = _time_launches(step, nbuf, steps, warmup)
    st = _stats(ms, b2b)
    return {
        "workload": name, "value": alg / (wall / steps) / 1e9, "unit": "GB/s", "ms_per_step": wall / steps * 1e3, "kernel_ms": st,
        "dtype": "f32 arithmetic, 8-bit out", "kernel": kern, "traffic_key": kind, "roofline": _roofline(0, alg, st, FP8_PEAK_TFLOPS, "TFLOP/s"),
    }


def bench_copy(steps, warmup):
    """Plain device-to-device copy of a known size (256 MiB read + 256 MiB written per launch): the calibration
    workload for the FETCH_SIZE / WRITE_SIZE counters behind `roofline.traffic`."""
    import torch

    dev = torch.device("cuda:0")
    n = 256 << 20
    srcs = [torch.randint(0, 255, (n,), dtype=torch.uint8, device=dev) for _ in range(3)]
    dsts = [torch.empty(n, dtype=torch.uint8, device=dev) for _ in range(3)]
    wall, ms, b2b = _time_launches(lambda i: dsts[i].copy_(srcs[i]), 3, steps, warmup)
    st = _stats(ms, b2b)
    return {
        "workload": f"copy {n} bytes device to device (torch copy kernel; {n} read + {n} written)",
        "value": 2 * n / (wall / steps) / 1e9, "unit": "GB/s", "ms_per_step": wall / steps * 1e3, "kernel_ms": st,
        "dtype": "u8", "roofline": _roofline(0, 2 * n, st, FP8_PEAK_TFLOPS, "TFLOP/s"),
    }


def _measured_traffic():
    """HBM bytes per launch measured with rocprofv3 counters (profiles/traffic.json), keyed by workload name."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get("bytes_per_launch", {})
    except (OSError, ValueError):
        return {}


def _traffic_key(rec):
    if "traffic_key" in rec:
        return rec["traffic_key"]
    head = rec["workload"].split(" (")[0].split(",")[0]  # e.g. "fp8_gemm gate_up M=4096 K=7168 N=36864"
    parts = head.split()
    if parts[0] == "group":
        return "quant_ue8m0" if "UE8M0" in rec["workload"] else "quant"
    return "_".join(x for x in parts if "=" not in x) + "".join("_" + x.replace("=", "") for x in parts if x.startswith("M="))


def _short(rec):
    """One compact row of the "also" list."""
    head = rec["workload"].split(" (")[0].replace("fp8_gemm ", "fp8 ").replace("int8_gemm ", "int8 ")
    ro = rec["roofline"]
    row = {"w": head, "ms": rec["kernel_ms"]["median"], "b2b": rec["kernel_ms"]["b2b"], "v": ro["achieved"], "u": ro["unit"],
           "bound": ro["bound"], "frac": ro["frac"]}
    if "kernel" in rec:
        row["kern"] = rec["kernel"]
    if ro.get("traffic"):
        row["traffic"] = ro["traffic"]
    if "operator_frac" in rec:
        row["operator_frac_same_call"] = rec["operator_frac"]
    if "streams" in rec:
        row["streams"] = [{"s": x["stream"], "on": x["operands"], "frac": x["frac"], "GHz": x["clock_GHz_if_pipe_full"]} for x in rec["streams"]]
    for k in ("cpu_baseline", "cpu_torch_native", "cpu_w8a16_shape"):
        if k in rec:
            row[k] = {"v": rec[k]["value"], "u": rec[k]["unit"], "cores": rec[k]["cores"], "kind": rec[k]["kind"],
                      "sample": rec[k]["sample"]}
    return row


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--quick", action="store_true", help="headline only (no 'also' list)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path is measured on ONE GPU; it contains no collective, and a run with --gpus N>1 "
              "is not provided (tokens shard by rows, weights by N or K, outside these kernels).", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from sglang_amd import _lib
    from sglang_amd.workloads import DSV3_MLA, DSV3_MLP, LLAMA3_8B

    _lib.lib()  # fail loudly if the HIP library is missing
    # spin the device up (clocks, allocator) before the first measurement
    _a = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0")
    _b = torch.empty_like(_a)
    _t = time.perf_counter()
    while time.perf_counter() - _t < 0.3:
        _b.copy_(_a)
        torch.cuda.synchronize()
    del _a, _b

    S, W, cpu = args.steps, args.warmup, not args.no_cpu
    also, quant = [], []
    wl = args.workload
    if wl in ("quant", "quant_ue8m0"):
        rec = bench_quant(S, W, wl == "quant_ue8m0", cpu)
    elif wl == "copy":
        rec = bench_copy(S, W)
    elif wl == "mfma_stream":
        rec = bench_mfma_stream(S, W)
    elif wl.startswith("fp8_ceiling"):
        parts = wl.split(":")
        K, N = DSV3_MLP["gate_up"]
        M = 4096
        if len(parts) == 4:
            M, K, N = int(parts[1]), int(parts[2]), int(parts[3])
        rec = bench_fp8_ceiling(M, K, N, S, W)
    elif wl == "silu_quant":
        rec = bench_silu_quant(S, W)
    elif wl in ("per_token_fp8", "per_token_int8", "per_tensor_fp8", "block_cast"):
        rec = bench_row_quant(wl, S, W)
    elif wl == "fp8_decode":
        K, N = DSV3_MLP["gate_up"]
        rec = bench_fp8_gemm("gate_up", 1, K, N, S, W, cpu)
    elif wl == "int8_gemm":
        K, N = LLAMA3_8B["gate_up"]
        rec = bench_int8_gemm("gate_up", 4096, K, N, S, W, cpu)
    elif wl.startswith("fp8_ue8m0:"):
        _, M, K, N = wl.split(":")
        rec = bench_fp8_ue8m0_gemm("shape", int(M), int(K), int(N), S, W)
    elif wl.startswith("fp8_linear:") or wl.startswith("fp8_linear2:"):
        kind, M, K, N = wl.split(":")
        rec = bench_fp8_linear(int(M), int(K), int(N), S, W, kind == "fp8_linear2")
    elif wl.startswith("fp8_grouped:"):
        _, E, m_per, K, N = wl.split(":")
        rec = bench_fp8_grouped_gemm(int(E), int(m_per), int(K), int(N), S, W)
    elif wl.startswith("fp8:") or wl.startswith("int8:"):
        kind, M, K, N = wl.split(":")
        fn = bench_fp8_gemm if kind == "fp8" else bench_int8_gemm
        rec = fn("shape", int(M), int(K), int(N), S, W, cpu)
    else:
        full = wl == "all" and not args.quick
        if full:
            # the bandwidth-bound quantizer is measured first: right after the MFMA-heavy GEMMs the chip's power state
            # makes a 60 us streaming kernel read ~15 % slow
            quant = [bench_quant(S, W, False, cpu), bench_quant(S, W, True, False)]
            also += [bench_row_quant(k, S, W) for k in ("per_token_fp8", "per_token_int8", "per_tensor_fp8", "block_cast")]
        K, N = DSV3_MLP["gate_up"]
        rec = bench_fp8_gemm("gate_up", 4096, K, N, S, W, cpu)
        if full:
            also.append(bench_fp8_ceiling(4096, K, N, S, W))
            also.append(bench_mfma_stream(S, W))
            also.append(bench_fp8_ue8m0_gemm("gate_up", 4096, K, N, S, W))
            # the same operator at decode and mid-M sizes: wave-split, streaming decode and three-stage kernels, each
            # with the scales applied by the MFMA
            for M in (1, 8, 128):
                also.append(bench_fp8_ue8m0_gemm("gate_up", M, K, N, S, W))
            also.append(bench_silu_quant(S, W))
            # expert GEMMs of DeepSeek-R1 (shapes of the reference's grouped-GEMM benchmark): prefill TP=8, prefill EP=16, decode EP=8
            for E, rows, Kg, Ng in ((256, 128, 7168, 512), (16, 512, 7168, 4096), (32, 4, 7168, 4096)):
                also.append(bench_fp8_grouped_gemm(E, rows, Kg, Ng, S, W))
            K, N = DSV3_MLP["down"]
            also.append(bench_fp8_gemm("down", 4096, K, N, S, W, False))
            for nm, (K, N) in DSV3_MLA.items():
                also.append(bench_fp8_gemm(nm, 4096, K, N, S, W, False))
            for M in (1, 8, 32, 128):
                for nm, (K, N) in DSV3_MLP.items():
                    also.append(bench_fp8_gemm(nm, M, K, N, S, W, False))
            also.append(bench_fp8_gemm("single_linear", 16, 7168, 2048, S, W, cpu, w8a16_cpu=cpu))
            # the whole decode linear bf16 -> bf16 in one call (quantizer inside the GEMM kernel) on the gate_up / down shapes
            for M in (1, 8):
                for nm, (K, N) in DSV3_MLP.items():
                    also.append(bench_fp8_linear(M, K, N, S, W, False))
            for M in (1, 256, 4096):
                for nm, (K, N) in LLAMA3_8B.items():
                    also.append(bench_int8_gemm(nm, M, K, N, S, W, with_cpu=(cpu and M == 4096 and nm == "gate_up")))

    traffic = _measured_traffic()
    for r in [rec] + also + quant:
        key = _traffic_key(r)
        if key in traffic:
            r["roofline"]["traffic"] = traffic[key]

    line = {
        "metric": METRIC, "value": rec["value"], "unit": rec["unit"], "n_gpus": 1, "steps": S, "warmup": W,
        "ms_per_step": rec["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": rec["dtype"], "data": DATA, "config": {"workload": rec["workload"]},
        "roofline": rec["roofline"], "kernel_ms": rec["kernel_ms"],
    }
    for k in ("kernel", "cpu_baseline", "cpu_torch_native", "operator_ms", "operator_frac", "streams"):
        if k in rec:
            line[k] = rec[k]
    if also:
        line["also"] = [_short(r) for r in also]
    if quant:
        # last in the line, so that a reader who only keeps the end of the output still has them
        line["quant"] = [{"workload": q["workload"], "value": q["value"], "unit": q["unit"], "kernel_ms": q["kernel_ms"],
                          "roofline": q["roofline"], **({"cpu_baseline": q["cpu_baseline"]} if "cpu_baseline" in q else {})}
                         for q in quant]
    print(json.dumps(r4(line), separators=(",", ":")))


if __name__ == "__main__":
    main()
