"""The shape grids of the reference's own operator tests, run through the operators under the reference's names.

sgl-kernel/tests/test_fp8_blockwise_gemm.py:62-85 runs fp8_blockwise_scaled_mm over M x N x K x out_dtype with operands
drawn uniformly from the whole e4m3fn range, scales ~ N(0, 1e-3) (either sign) laid out M-major, and accepts
rtol 0.02 / atol 1 against scale-then-multiply in fp32; sgl-kernel/tests/test_int8_gemm.py:20-49 runs int8_scaled_mm over
M x N x K x bias x out_dtype with int8(N(0, 5)) operands, N(0, 1) scales of either sign and a bias of N(0, 10).

The same grids, operand distributions and (for FP8) the same criterion are used here; the comparison values are built
with torch on the GPU, as the reference's tests build theirs, and - because that is one GPU library checking another - every
FP8 case is also held to the CPU oracle on a sample of token rows over all channels, under the criterion of
tests/fp8_tolerance.py.  FP8 is floating point, so the reference's tolerance
applies; the INT8 result is held to the bits: exact integer accumulators (an fp64 matmul is exact at these sizes), then the
epilogue f32(acc) * (sb[n] * sa[m]) + bias, each step rounded once.  Cases above 2^36 multiply-accumulates are left to
the curated full-size tests (tests/test_gpu_fp8_gemm.py, tests/test_gpu_int8_gemm.py, tests/test_gpu_config_shapes.py).
"""
import pytest
import torch

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
MAX_MACS = 1 << 36

FP8_M = [1, 3, 5, 127, 128, 512, 1024, 4096]
FP8_N = [128, 512, 1024, 4096, 8192, 14080]
FP8_K = [512, 1024, 4096, 8192, 14080, 16384]
INT8_M = [1, 16, 32, 64, 128, 512, 1024, 4096, 8192]
INT8_N = [16, 128, 512, 1024, 4096, 8192, 16384]
INT8_K = [512, 1024, 4096, 8192, 16384]


def _m_major(t):
    return t.t().contiguous().t()


@pytest.mark.parametrize("N", FP8_N)
@pytest.mark.parametrize("K", FP8_K)
def test_fp8_blockwise_scaled_mm_reference_grid(gpu, oracle, N, K):
    from fp8_tolerance import check_fp8_gemm
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    g = torch.Generator(device=gpu).manual_seed(N * 31 + K)
    w = ((torch.rand(N, K, generator=g, device=gpu) - 0.5) * 2 * 448.0).clamp(-448, 448).to(FP8)
    sb = _m_major(torch.randn(K // 128, N // 128, generator=g, device=gpu) * 0.001)  # shaped like mat_b: [K / 128, N / 128]
    wb = w.float() * sb.t().repeat_interleave(128, 0).repeat_interleave(128, 1)
    w_cpu = sw_cpu = None
    ran = 0
    for M in FP8_M:
        if M * N * K > MAX_MACS:
            continue
        print(f"case fp8 M={M} N={N} K={K}", flush=True)
        a = ((torch.rand(M, K, generator=g, device=gpu) - 0.5) * 2 * 448.0).clamp(-448, 448).to(FP8)
        sa = _m_major(torch.randn(M, K // 128, generator=g, device=gpu) * 0.001)
        want32 = (a.float() * sa.repeat_interleave(128, 1)) @ wb.t()
        for out_dtype in (torch.bfloat16, torch.float16):
            out = fp8_blockwise_scaled_mm(a, w.t(), sa, sb, out_dtype)
            assert out.dtype == out_dtype and tuple(out.shape) == (M, N)
            torch.testing.assert_close(out, want32.to(out_dtype), rtol=0.02, atol=1)
        # the oracle on up to eight token rows (first, last, tile borders) over all channels; out is the fp16 result
        rows = sorted({0, M - 1, M // 2, min(M - 1, 127), min(M - 1, 128), min(M - 1, 255), min(M - 1, 256), M // 3})
        if w_cpu is None:
            w_cpu, sw_cpu = w.cpu(), sb.t().contiguous().cpu()
        idx = torch.tensor(rows, device=gpu)
        ref, mag = oracle.fp8_blockwise_mm(a[idx].cpu().contiguous(), w_cpu, sa[idx].cpu().contiguous(), sw_cpu, torch.float32, want_abs=True)
        check_fp8_gemm(out[idx], ref, mag, f"grid M={M} N={N} K={K}")
        ran += 1
    assert ran >= 5  # every (N, K) pair runs at least the five smallest token counts


@pytest.mark.parametrize("N", INT8_N)
@pytest.mark.parametrize("K", INT8_K)
def test_int8_scaled_mm_reference_grid(gpu, N, K):
    from sglang_amd.sgl_kernel import int8_scaled_mm

    g = torch.Generator(device=gpu).manual_seed(N * 17 + K)
    w = (torch.randn(N, K, generator=g, device=gpu) * 5).round().clamp(-128, 127).to(torch.int8)
    sb = torch.randn(N, generator=g, device=gpu)
    w64 = w.double()
    ran = 0
    for M in INT8_M:
        if M * N * K > MAX_MACS:
            continue
        print(f"case int8 M={M} N={N} K={K}", flush=True)
        a = (torch.randn(M, K, generator=g, device=gpu) * 5).round().clamp(-128, 127).to(torch.int8)
        sa = torch.randn(M, generator=g, device=gpu)
        acc = (a.double() @ w64.t()).to(torch.float32)            # exact integers, rounded once to fp32 like (float)acc
        scaled = acc * (sb.view(1, N) * sa.view(M, 1))            # f32(acc) * (sb * sa), each product rounded once
        for out_dtype in (torch.bfloat16, torch.float16):
            bias = (torch.randn(N, generator=g, device=gpu) * 10).to(out_dtype)
            for b in (None, bias):
                out = int8_scaled_mm(a, w.t(), sa, sb, out_dtype, b)
                want = (scaled if b is None else scaled + b.float().view(1, N)).to(out_dtype)
                assert out.dtype == out_dtype and tuple(out.shape) == (M, N)
                assert torch.equal(out.view(torch.int16), want.view(torch.int16)), (M, N, K, out_dtype, b is not None)
        ran += 1
    assert ran >= 5  # every (N, K) pair runs at least the five smallest token counts


# ---- sgl-kernel/tests/test_per_token_group_quant_8bit.py:22-59: tokens x hidden x group x {fp8, int8} x four scale layouts,
# through sglang_per_token_group_quant_8bit(enable_v2=True) as that test calls it.  There the CUDA kernel is compared with
# the Triton kernel under a tolerance; here codes and scales must equal the CPU oracle's bit for bit, so the inputs are
# capped at 2^21 elements per case (the full-size configuration has its own test in tests/test_gpu_group_quant.py).
QUANT_TOKENS = [1, 4, 16, 64, 127, 128, 512, 1024, 4096, 8192]
QUANT_HIDDEN = [128, 256, 384, 512, 1024, 1536, 1664, 2048, 4096, 7168, 16384]
QUANT_LAYOUTS = ["row", "col", "col_aligned", "ue8m0"]


@pytest.mark.parametrize("hidden", QUANT_HIDDEN)
@pytest.mark.parametrize("group", [16, 32, 64, 128])
def test_per_token_group_quant_8bit_reference_grid(gpu, oracle, hidden, group):
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_8bit
    from sglang_amd.workloads import make_activation

    ran = 0
    for tokens in QUANT_TOKENS:
        if tokens * hidden > (1 << 21):
            continue
        x = make_activation(tokens, hidden, seed=tokens * 13 + hidden + group, zero_group_frac=0.02, group=group)
        xg = x.to(gpu)
        for dst in (FP8, torch.int8):
            for layout in QUANT_LAYOUTS:
                if (layout == "ue8m0" and group != 128) or (dst == torch.int8 and layout != "row"):
                    continue  # the combinations the reference's test skips too
                print(f"case quant tokens={tokens} hidden={hidden} group={group} {dst} {layout}", flush=True)
                q, s = sglang_per_token_group_quant_8bit(
                    xg, group, dst, column_major_scales=layout != "row", scale_tma_aligned=layout in ("col_aligned", "ue8m0"),
                    scale_ue8m0=layout == "ue8m0", enable_v2=True)
                q_o, s_o = oracle.group_quant(x, group, mode="mul", layout=layout, dst_dtype=dst)
                assert q.dtype == dst and tuple(s.shape) == tuple(s_o.shape) and s.dtype == s_o.dtype
                assert torch.equal(q.cpu().view(torch.uint8), q_o.view(torch.uint8)), (tokens, hidden, group, dst, layout)
                if layout == "ue8m0":
                    n = 4 * s.shape[1]
                    assert torch.equal(oracle.unpack_ue8m0(s.cpu(), n), oracle.unpack_ue8m0(s_o, n))
                else:
                    assert torch.equal(s.cpu().contiguous().view(torch.int32), s_o.contiguous().view(torch.int32))
                ran += 1
    assert ran >= 12


# ---- sgl-kernel/tests/test_per_token_quant_fp8.py:37-53 and test_per_tensor_quant_fp8.py:39-66: fp16 inputs uniform in
# [0, 1), tokens x hidden incl. 1368 (rows of 171 16-byte vectors); per-tensor both dynamic and with a given scale.  Those
# tests re-derive the codes from the kernel's own scale under a tolerance; here codes and scales equal the oracle's bits.
@pytest.mark.parametrize("tokens", [128, 256, 512])
@pytest.mark.parametrize("hidden", [512, 1368, 2048, 4096])
def test_per_token_and_per_tensor_quant_fp8_reference_grid(gpu, oracle, tokens, hidden):
    from sglang_amd.sgl_kernel import sgl_per_tensor_quant_fp8, sgl_per_token_quant_fp8

    g = torch.Generator().manual_seed(tokens + hidden)
    x = torch.rand(tokens, hidden, generator=g).to(torch.float16)
    xg = x.to(gpu)
    q = torch.empty(tokens, hidden, dtype=FP8, device=gpu)
    s = torch.zeros(tokens, dtype=torch.float32, device=gpu)
    sgl_per_token_quant_fp8(xg, q, s)
    q_o, s_o = oracle.per_token_quant_fp8(x)
    assert torch.equal(q.cpu().view(torch.uint8), q_o.view(torch.uint8)) and torch.equal(s.cpu().view(torch.int32), s_o.view(-1).view(torch.int32))
    for given in (None, torch.rand(1, generator=g)):
        scale = torch.zeros(1, dtype=torch.float32, device=gpu) if given is None else given.to(gpu)
        sgl_per_tensor_quant_fp8(xg, q, scale, given is not None)
        q_o, s_o = oracle.per_tensor_quant_fp8(x, given)
        assert torch.equal(q.cpu().view(torch.uint8), q_o.view(torch.uint8)), (tokens, hidden, given)
        assert torch.equal(scale.cpu().view(torch.int32), s_o.view(torch.int32))


# ---- sgl-kernel/tests/test_fp8_gemm.py:39-45: fp8_scaled_mm over M x N x K x bias x out_dtype, full-range codes, per-token
# and per-channel scales ~ N(0, 1e-3), bias ~ N(0, 1) in the output type; the reference's formula and its rtol 0.02 / atol 1.
@pytest.mark.parametrize("N", [16, 128, 512, 1024, 4096])
@pytest.mark.parametrize("K", [512, 1024, 4096, 8192, 16384])
def test_fp8_scaled_mm_reference_grid(gpu, oracle, N, K):
    from fp8_tolerance import check_fp8_gemm
    from sglang_amd.sgl_kernel import fp8_scaled_mm

    g = torch.Generator(device=gpu).manual_seed(N * 7 + K)
    w = ((torch.rand(N, K, generator=g, device=gpu) - 0.5) * 2 * 448.0).clamp(-448, 448).to(FP8)
    sb = torch.randn(N, generator=g, device=gpu) * 0.001
    w32 = w.float()
    for M in (1, 128, 512, 1024, 4096):
        print(f"case fp8_scaled_mm M={M} N={N} K={K}", flush=True)
        a = ((torch.rand(M, K, generator=g, device=gpu) - 0.5) * 2 * 448.0).clamp(-448, 448).to(FP8)
        sa = torch.randn(M, generator=g, device=gpu) * 0.001
        scaled = (a.float() @ w32.t()) * sa.view(-1, 1) * sb.view(1, -1)
        for out_dtype in (torch.bfloat16, torch.float16):
            bias = torch.randn(N, generator=g, device=gpu).to(out_dtype)
            for b in (None, bias):
                out = fp8_scaled_mm(a, w.t(), sa, sb, out_dtype, b)
                want = scaled.to(out_dtype) if b is None else scaled.to(out_dtype) + b.view(1, -1)
                torch.testing.assert_close(out, want, rtol=0.02, atol=1)
        # the last result (fp16, with bias) against the CPU oracle on a sample of token rows
        rows = sorted({0, M - 1, M // 2, min(M - 1, 255), min(M - 1, 256), M // 3})
        idx = torch.tensor(rows, device=gpu)
        ref, mag = oracle.fp8_scaled_mm(a[idx].cpu().contiguous(), w.cpu(), sa[idx].cpu().contiguous(), sb.cpu(), torch.float32, None, want_abs=True)
        check_fp8_gemm(out[idx], ref + bias.float().cpu()[None, :], mag, f"fp8_scaled_mm grid M={M} N={N} K={K}")


# ---- python/sglang/test/test_block_fp8.py:326-398 (TestW8A8BlockFP8Matmul), both of its grids: the generic one with ragged
# N = 7748 and K = 3884 / 5120 / 256 and fp32 / fp16 / bf16 outputs, and the DeepSeek-V3 one; full-range codes, scales
# uniform in [0, 1e-2), row-major token scales, through fp8_kernel.w8a8_block_fp8_matmul; its criterion
# mean|out - ref| / mean|ref| < 0.001 against the broadcast-scale fp32 product.
GENERIC_NK = [(N, K) for N in (128, 512, 1024, 4096, 7748, 13824) for K in (256, 4096, 5120, 3884, 13824)]
DSV3_NK = [(2112, 7168), (1536, 7168), (3072, 1536), (24576, 7168), (4096, 512), (7168, 2048), (4608, 7168), (512, 7168),
           (7168, 2304), (7168, 512)]


def _block_matmul_case(gpu, oracle, N, K, Ms, out_dtypes):
    from fp8_tolerance import check_fp8_gemm
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul

    g = torch.Generator(device=gpu).manual_seed(N + K)
    nt, kt = -(-N // 128), -(-K // 128)
    w = ((torch.rand(N, K, generator=g, device=gpu) - 0.5) * 2 * 448.0).clamp(-448, 448).to(FP8)
    Bs = torch.rand(nt, kt, generator=g, device=gpu) * 1e-2
    wb = w.float() * Bs.repeat_interleave(128, 0)[:N].repeat_interleave(128, 1)[:, :K]
    for M in Ms:
        print(f"case block matmul M={M} N={N} K={K}", flush=True)
        a = ((torch.rand(M, K, generator=g, device=gpu) - 0.5) * 2 * 448.0).clamp(-448, 448).to(FP8)
        As = torch.rand(M, kt, generator=g, device=gpu) * 1e-2
        ref32 = (a.float() * As.repeat_interleave(128, 1)[:, :K]) @ wb.t()
        for out_dtype in out_dtypes:
            out = w8a8_block_fp8_matmul(a, w, As, Bs, [128, 128], out_dtype)
            ref = ref32.to(out_dtype).float()
            assert out.dtype == out_dtype and tuple(out.shape) == (M, N)
            assert float((out.float() - ref).abs().mean() / ref.abs().mean()) < 0.001, (M, N, K, out_dtype)
        # the last result against the CPU oracle on a sample of token rows (ragged N and K included)
        rows = sorted({0, M - 1, M // 2, min(M - 1, 255), min(M - 1, 256), M // 3})
        idx = torch.tensor(rows, device=gpu)
        want, mag = oracle.fp8_blockwise_mm(a[idx].cpu().contiguous(), w.cpu(), As[idx].cpu().contiguous(), Bs.cpu(), torch.float32, want_abs=True)
        check_fp8_gemm(out[idx], want, mag, f"block matmul grid M={M} N={N} K={K}")


@pytest.mark.parametrize("N,K", GENERIC_NK)
def test_w8a8_block_fp8_matmul_generic_grid(gpu, oracle, N, K):
    _block_matmul_case(gpu, oracle, N, K, [1, 7, 83, 512, 2048], [torch.float32, torch.half, torch.bfloat16])


@pytest.mark.parametrize("N,K", DSV3_NK)
def test_w8a8_block_fp8_matmul_deepseek_grid(gpu, oracle, N, K):
    _block_matmul_case(gpu, oracle, N, K, [64, 128, 512, 1024, 4096], [torch.bfloat16])


# ---- python/sglang/test/test_block_fp8.py:51-92 (TestPerTokenGroupQuantFP8) and :118-158 (TestStaticQuantFP8): inputs uniform
# in [0, 1) in fp16 / bf16 / fp32, tokens x hidden incl. 5120 and 13824, groups of 64 .. 512.  The reference compares with a
# torch restatement under rtol 0.15; here the codes and scales equal the oracle's bits (cases above 2^23 elements left out).
@pytest.mark.parametrize("dtype", [torch.half, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("hidden", [512, 4096, 5120, 13824])
def test_python_level_quantizer_grids(gpu, oracle, dtype, hidden):
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8, static_quant_fp8

    for tokens in (7, 83, 2048):
        if tokens * hidden > (1 << 23):
            continue
        g = torch.Generator().manual_seed(tokens + hidden)
        x = torch.rand(tokens, hidden, generator=g).to(dtype)
        xg = x.to(gpu)
        for group in (64, 128, 256, 512):
            print(f"case group quant tokens={tokens} hidden={hidden} group={group} {dtype}", flush=True)
            q, s = per_token_group_quant_fp8(xg, group)
            q_o, s_o = oracle.group_quant(x, group, mode="rcp", layout="row")
            assert tuple(s.shape) == (tokens, hidden // group)
            assert torch.equal(q.cpu().view(torch.uint8), q_o.view(torch.uint8)), (tokens, hidden, group, dtype)
            assert torch.equal(s.cpu().view(torch.int32), s_o.view(torch.int32))
        x_s = (x.float().max() / 448.0).reshape(1)
        q, s = static_quant_fp8(xg, x_s.to(gpu))
        q_o, _ = oracle.per_tensor_quant_fp8(x, x_s)
        assert torch.equal(q.cpu().view(torch.uint8), q_o.view(torch.uint8)), (tokens, hidden, dtype, "static")
        assert float(s) == float(x_s)
