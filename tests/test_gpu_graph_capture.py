"""The operators under HIP graph capture: quantize -> blockwise FP8 GEMM -> INT8 GEMM recorded once on a side stream and
replayed with new input contents.

What this pins: nothing on the path synchronizes, allocates outside torch's capture-aware allocator or depends on host
state at replay time (the reference runs these operators inside its decode graphs,
python/sglang/srt/model_executor/cuda_graph_runner.py:452-540).  Every replay is compared with the eager result of the
same inputs (bit for bit: same kernels, deterministic reduce order) and the first one with the CPU oracle.  Replays are
separated by eager work and synchronizations, and the graph holds no memset node of its own (split-K partial sums need no
clearing).  Shapes cover the wave-split decode plan, a split-K decode plan (workspace from torch inside the capture), a mid-M
plan with re-laid-out token scales, and an unsplit plan.
"""
import pytest
import torch

from fp8_tolerance import check_fp8_gemm
from sglang_amd.workloads import make_activation, make_fp8_weight, make_int8_weight

pytestmark = pytest.mark.gpu


def _linear_chain(x, w_q, w_s, wi_q, wi_s):
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8, w8a8_block_fp8_matmul
    from sglang_amd.int8_kernel import per_token_quant_int8
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm, int8_scaled_mm

    x_q, x_s = per_token_group_quant_fp8(x, 128, column_major_scales=True)
    y = fp8_blockwise_scaled_mm(x_q, w_q.t(), x_s, w_s.t(), torch.bfloat16)       # [M, N1]
    x_q2, x_s2 = per_token_group_quant_fp8(x, 128)                                   # row-major scales: re-layout path
    y2 = w8a8_block_fp8_matmul(x_q2, w_q, x_s2, w_s, [128, 128], torch.bfloat16)
    a_q, a_s = per_token_quant_int8(y)
    z = int8_scaled_mm(a_q, wi_q.t(), a_s, wi_s, torch.bfloat16)                    # [M, N2]
    return x_q, x_s, y, y2, z


@pytest.mark.parametrize("M", [4, 12, 48, 300])  # wave-split decode, split-K streaming decode, mid-M, unsplit
def test_capture_and_replay_matches_eager(gpu, oracle, M):
    from sglang_amd import _lib

    K, N1, N2 = 2048, 1024, 512
    plan = _lib.gemm_plan("fp8", M, N1, K)
    print(f"case M={M}: fp8 {plan}  int8 {_lib.gemm_plan('int8', M, N2, N1)}", flush=True)
    w_q, w_s = make_fp8_weight(N1, K, seed=11)
    wi_q, wi_s = make_int8_weight(N2, N1, seed=12)
    w_q, w_s, wi_q, wi_s = w_q.to(gpu), w_s.to(gpu), wi_q.to(gpu), wi_s.to(gpu)
    inputs = [make_activation(M, K, seed=100 + i) for i in range(4)]
    static_x = inputs[0].to(gpu).clone()

    stream = torch.cuda.Stream()  # default priority
    with torch.cuda.stream(stream):
        for _ in range(2):  # warm up allocator, lazy initialisation and operator registration outside the capture
            _linear_chain(static_x, w_q, w_s, wi_q, wi_s)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            static_out = _linear_chain(static_x, w_q, w_s, wi_q, wi_s)
    torch.cuda.synchronize()

    for i, x in enumerate(inputs[1:] + inputs[:1]):
        static_x.copy_(x.to(gpu))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in static_out]
        # eager work between replays, then the eager result of the same input
        want = _linear_chain(x.to(gpu), w_q, w_s, wi_q, wi_s)
        torch.cuda.synchronize()
        for name, g_, w_ in zip(("x_q", "x_s", "y", "y2", "z"), got, want):
            assert torch.equal(g_.view(torch.uint8) if g_.dtype == torch.float8_e4m3fn else g_,
                               w_.view(torch.uint8) if w_.dtype == torch.float8_e4m3fn else w_), (i, name)
        if i == 0:
            q_o, s_o = oracle.group_quant(x, 128, mode="div", layout="col")
            assert torch.equal(got[0].cpu().view(torch.uint8), q_o.view(torch.uint8)) and torch.equal(got[1].cpu(), s_o)
            ref, mag = oracle.fp8_blockwise_mm(q_o, w_q.cpu(), s_o, w_s.cpu(), torch.float32, want_abs=True)
            check_fp8_gemm(got[2], ref, mag, f"replay {i}")


@pytest.mark.parametrize("M", [2, 12, 48])  # wave-split decode, split-K streaming decode, mid-M: each with MFMA-applied scales
def test_packed_scale_linear_replays(gpu, M):
    """Quantizer with packed UE8M0 scales -> GEMM that takes the packed words on both operands, captured and replayed with
    new inputs; every replay equals the eager result of the same input bit for bit."""
    from sglang_amd import _lib
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8, w8a8_block_fp8_matmul_deepgemm
    from sglang_amd.fp8_utils import requant_weight_ue8m0

    K, N = 2048, 1024
    print(f"case M={M}: {_lib.gemm_plan('fp8', M, N, K)}", flush=True)
    w_q, w_s = make_fp8_weight(N, K, seed=21)
    w2, sw = requant_weight_ue8m0(w_q.to(gpu), w_s.to(gpu), [128, 128])

    def chain(x):
        x_q, x_s = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True,
                                                    enable_v2=True)
        return x_q, x_s, w8a8_block_fp8_matmul_deepgemm(x_q, w2, x_s, sw, [128, 128], torch.bfloat16)

    inputs = [make_activation(M, K, seed=200 + i) for i in range(3)]
    static_x = inputs[0].to(gpu).clone()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(2):
            chain(static_x)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            static_out = chain(static_x)
    torch.cuda.synchronize()
    for i, x in enumerate(inputs[1:] + inputs[:1]):
        static_x.copy_(x.to(gpu))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in static_out]
        want = chain(x.to(gpu))
        torch.cuda.synchronize()
        assert torch.equal(got[0].view(torch.uint8), want[0].view(torch.uint8)), i
        assert torch.equal(got[1], want[1]), i
        assert torch.equal(got[2].view(torch.int16), want[2].view(torch.int16)), i
        assert bool(torch.isfinite(got[2]).all())


def test_grouped_gemm_replays_with_new_routing(gpu, oracle):
    """The grouped FP8 GEMM inside a graph: problem sizes and expert offsets are device data, so a replay with a different
    routing (other rows per expert, experts gaining and losing 256-row tiles) rebuilds its tile schedule on the device.
    Each replay is compared with the eager call on the same data and the first one with the oracle."""
    from sglang_amd.sgl_kernel import es_fp8_blockwise_scaled_grouped_mm

    E, N, K, T = 6, 512, 1024, 900
    g = torch.Generator().manual_seed(3)
    a = ((torch.rand(T, K, generator=g) - 0.5) * 896).clamp(-448, 448).to(torch.float8_e4m3fn)
    w = ((torch.rand(E, N, K, generator=g) - 0.5) * 896).clamp(-448, 448).to(torch.float8_e4m3fn)
    sa = torch.rand(T, K // 128, generator=g) * 1e-2 + 1e-4
    sw = torch.rand(E, N // 128, K // 128, generator=g) * 1e-2 + 1e-4
    routings = [[150, 150, 150, 150, 150, 150], [700, 0, 1, 60, 139, 0], [0, 0, 0, 0, 0, 900], [3, 290, 7, 300, 44, 256]]
    a_d, w_d, sa_d, sw_d = a.to(gpu), w.to(gpu).transpose(1, 2), sa.to(gpu), sw.to(gpu).transpose(1, 2)
    strides = torch.full((E,), K, dtype=torch.int64, device=gpu)
    ws = torch.empty(8 << 20, dtype=torch.uint8, device=gpu)

    def tensors(sizes):
        offs = [sum(sizes[:e]) for e in range(E)]
        return (torch.tensor([[m, N, K] for m in sizes], dtype=torch.int32, device=gpu),
                torch.tensor(offs, dtype=torch.int32, device=gpu), offs)

    static_ps, static_eo, _ = tensors(routings[0])
    static_out = torch.zeros(T, N, dtype=torch.bfloat16, device=gpu)

    def run(out, ps, eo):
        es_fp8_blockwise_scaled_grouped_mm(out, a_d, w_d, sa_d, sw_d, strides, strides, strides, ps, eo, ws)

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        run(static_out, static_ps, static_eo)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            run(static_out, static_ps, static_eo)
    torch.cuda.synchronize()

    for i, sizes in enumerate(routings[1:] + routings[:1]):
        ps, eo, offs = tensors(sizes)
        static_ps.copy_(ps)
        static_eo.copy_(eo)
        static_out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = static_out.clone()
        want = torch.zeros_like(got)
        run(want, ps, eo)  # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(got, want), (i, sizes)
        if i == 0:
            for e, (m, r0) in enumerate(zip(sizes, offs)):
                if m:
                    ref, mag = oracle.fp8_blockwise_mm(a[r0:r0 + m], w[e], sa[r0:r0 + m], sw[e], torch.float32, want_abs=True)
                    check_fp8_gemm(got[r0:r0 + m], ref, mag, f"replay {e}")


@pytest.mark.parametrize("M,N,K", [(4, 1024, 2048), (12, 1024, 2048), (13, 53248, 1152), (48, 1024, 2048)])
def test_linear_methods_replay(gpu, M, N, K):
    """The linear layers as the reference's methods call them - both block-FP8 wrappers (one C-ABI call each: the quantizer in the
    streaming kernel's prologue, producer waves of the mid-M kernel, or a quantizer launch), the per-token FP8 linear and the INT8
    linear - captured once and replayed with new inputs: every replay equals the eager result of the same input bit for bit."""
    from sglang_amd import _lib
    from sglang_amd.fp8_utils import apply_fp8_linear, cutlass_w8a8_block_fp8_linear_with_fallback, triton_w8a8_block_fp8_linear
    from sglang_amd.w8a8_int8 import apply_w8a8_int8_linear

    print(f"case M={M}: {_lib.block_linear_plan(M, N, K)}", flush=True)
    N2 = 512
    w_q, w_s = make_fp8_weight(N, K, seed=31)
    wi_q, wi_s = make_int8_weight(N2, K, seed=32)
    w_q, w_s, wi_q, wi_s = w_q.to(gpu), w_s.to(gpu), wi_q.to(gpu).t(), wi_s.to(gpu)
    wc = w_q[:N2].t()  # [K, N2] column-major view for the per-token FP8 linear
    sc = torch.rand(N2, device=gpu) * 1e-2 + 1e-4
    bias = torch.randn(N2, device=gpu).to(torch.bfloat16)

    def chain(x):
        return (cutlass_w8a8_block_fp8_linear_with_fallback(x, w_q, [128, 128], w_s),
                triton_w8a8_block_fp8_linear(x, w_q, [128, 128], w_s),
                apply_fp8_linear(x, wc, sc, bias=bias),
                apply_w8a8_int8_linear(x, wi_q, wi_s, bias))

    inputs = [make_activation(M, K, seed=300 + i) for i in range(3)]
    static_x = inputs[0].to(gpu).clone()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(2):
            chain(static_x)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            static_out = chain(static_x)
    torch.cuda.synchronize()
    for i, x in enumerate(inputs[1:] + inputs[:1]):
        static_x.copy_(x.to(gpu))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in static_out]
        want = chain(x.to(gpu))
        torch.cuda.synchronize()
        for name, g_, w_ in zip(("cutlass-style", "triton-style", "per-token fp8", "int8"), got, want):
            assert torch.equal(g_.view(torch.int16), w_.view(torch.int16)), (i, name)
            assert bool(torch.isfinite(g_).all())
