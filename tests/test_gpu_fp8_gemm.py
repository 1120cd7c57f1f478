"""GPU parity of the blockwise-scaled FP8 GEMM (both reference entry points) against the CPU oracle.

Tolerance (floating point, written out in tests/fp8_tolerance.py with the measurements behind it):
|out - ref| <= 1e-2 * |ref| + 1e-4 * mag, mag = sum_k |a*b*sa*sb|; at least 99.5 % of the elements of every case must meet
the pure 1e-2 criterion.  The reference's own, looser, criteria (rtol 0.02 / atol 1 and mean-abs-rel < 1e-3) are asserted too.
"""
import pytest
import torch

from fp8_tolerance import FP8_MAG_TOL, FP8_MAG_TOL_CONFIG, check_fp8_gemm
from sglang_amd.workloads import cdiv, make_activation, make_fp8_weight

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def _rand_fp8(shape, g):
    return ((torch.rand(*shape, generator=g) - 0.5) * 2 * 448.0).clamp(-448, 448).to(FP8)


def _check(out, ref, mag, what="", mag_tol=FP8_MAG_TOL, min_pure=0.995):
    out_dtype = out.dtype
    stats = check_fp8_gemm(out, ref, mag, what, mag_tol, min_pure)
    print(f"{what}: {stats}", flush=True)
    out = out.float().cpu()
    # the reference's own acceptance tests; both compare with a reference already cast to the output dtype
    ref_cast = ref.to(out_dtype).float()
    torch.testing.assert_close(out, ref_cast, rtol=0.02, atol=1.0)
    denom = float(ref_cast.abs().mean())
    if denom > 0:
        assert float((out - ref_cast).abs().mean()) / denom < 1e-3
    return stats


# (M, N, K): every tile configuration (16/32/64/128/256 token tiles), split-K and non-split,
# M tails, and the DeepSeek-V3 projection shapes at reduced size.
ALIGNED_SHAPES = [
    (1, 128, 128), (1, 512, 7168), (3, 256, 512), (5, 1024, 1024), (16, 2048, 7168), (17, 384, 2304),
    (32, 1536, 1536), (33, 512, 512), (64, 4096, 512), (83, 7168, 256), (127, 128, 4096), (128, 2176, 1024),
    (130, 640, 896), (512, 4608, 512), (1024, 512, 1024), (1100, 1536, 384), (2048, 256, 2048),
]


@pytest.mark.parametrize("M,N,K", ALIGNED_SHAPES)
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_sgl_kernel_fp8_blockwise_scaled_mm(gpu, oracle, M, N, K, out_dtype):
    """Operand layouts of sgl-kernel/tests/test_fp8_blockwise_gemm.py:62-81: mat_b and both scale
    tensors are column-major views."""
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    print(f"case M={M} N={N} K={K} {out_dtype}", flush=True)
    g = torch.Generator().manual_seed(M * 31 + N * 7 + K)
    a, w = _rand_fp8((M, K), g), _rand_fp8((N, K), g)
    scale_a = (torch.randn(M, K // 128, generator=g) * 1e-3).t().contiguous().t()
    scale_b = (torch.randn(K // 128, N // 128, generator=g) * 1e-3).t().contiguous().t()
    assert scale_a.stride(0) == 1 or M == 1 or K == 128
    out = fp8_blockwise_scaled_mm(a.to(gpu), w.to(gpu).t(), scale_a.to(gpu).t().contiguous().t(),
                                  scale_b.to(gpu).t().contiguous().t(), out_dtype)
    assert out.dtype == out_dtype and tuple(out.shape) == (M, N)
    ref, mag = oracle.fp8_blockwise_mm(a, w, scale_a, scale_b.t(), torch.float32, want_abs=True)
    _check(out, ref, mag, f"M={M} N={N} K={K}")


RAGGED_SHAPES = [(7, 1088, 512), (83, 7748, 256), (16, 576, 7168), (64, 128, 3884), (130, 200, 300),
                 (1, 1088, 3884), (256, 576, 1024)]


@pytest.mark.parametrize("M,N,K", RAGGED_SHAPES)
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_w8a8_block_fp8_matmul_ragged(gpu, oracle, M, N, K, out_dtype):
    """python/sglang/test/test_block_fp8.py:328-414: N and K need not be multiples of 128, scales have
    ceil-divided shapes, B is the row-major weight."""
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul

    print(f"case M={M} N={N} K={K} {out_dtype}", flush=True)
    g = torch.Generator().manual_seed(M + N + K)
    a, w = _rand_fp8((M, K), g), _rand_fp8((N, K), g)
    As = torch.rand(M, cdiv(K, 128), generator=g) * 1e-2
    Bs = torch.rand(cdiv(N, 128), cdiv(K, 128), generator=g) * 1e-2
    out = w8a8_block_fp8_matmul(a.to(gpu), w.to(gpu), As.to(gpu), Bs.to(gpu), [128, 128], out_dtype)
    assert out.dtype == out_dtype and tuple(out.shape) == (M, N)
    ref, mag = oracle.fp8_blockwise_mm(a, w, As, Bs, torch.float32, want_abs=True)
    _check(out, ref, mag, f"M={M} N={N} K={K}")


def test_batched_leading_dims_and_default_dtype(gpu, oracle):
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul

    g = torch.Generator().manual_seed(3)
    a, w = _rand_fp8((2, 5, 256), g), _rand_fp8((384, 256), g)
    As = torch.rand(2, 5, 2, generator=g) * 1e-3
    Bs = torch.rand(3, 2, generator=g) * 1e-3
    out = w8a8_block_fp8_matmul(a.to(gpu), w.to(gpu), As.to(gpu), Bs.to(gpu), [128, 128])
    assert out.dtype == torch.float16 and tuple(out.shape) == (2, 5, 384)
    ref, mag = oracle.fp8_blockwise_mm(a.view(10, 256), w, As.view(10, 2), Bs, torch.float32, want_abs=True)
    _check(out.view(10, 384), ref, mag)


def test_exact_integer_case(gpu):
    """Integer-valued codes and power-of-two scales: every product, block sum and promotion is exact in
    fp32, whatever the summation order, so the GPU must reproduce integer arithmetic exactly.  Catches a
    transposed operand, a dropped or doubled K block and a wrong scale index."""
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul

    g = torch.Generator().manual_seed(4)
    for M, N, K in [(9, 384, 640), (300, 256, 1152), (16, 1024, 4096)]:
        ai = torch.randint(-8, 9, (M, K), generator=g)
        wi = torch.randint(-8, 9, (N, K), generator=g)
        sa = torch.exp2(torch.randint(-3, 4, (M, K // 128), generator=g).float())
        sw = torch.exp2(torch.randint(-3, 4, (N // 128, K // 128), generator=g).float())
        out = w8a8_block_fp8_matmul(ai.float().to(FP8).to(gpu), wi.float().to(FP8).to(gpu), sa.to(gpu), sw.to(gpu),
                                    [128, 128], torch.float32)
        want = torch.zeros(M, N, dtype=torch.float64)
        for kb in range(K // 128):
            part = (ai[:, kb * 128:(kb + 1) * 128] @ wi[:, kb * 128:(kb + 1) * 128].T).double()
            want += part * sa[:, kb:kb + 1].double() * sw[:, kb].double().repeat_interleave(128)[None, :]
        assert torch.equal(out.cpu().double(), want), (M, N, K)


@pytest.mark.parametrize("M", [16, 128])
def test_quantize_then_gemm_single_linear(gpu, oracle, M):
    """The single-linear configuration (K=7168 -> N=2048): activations with outliers are quantized on the
    GPU (column-major scales, as the caller in fp8_utils.py:184-214 asks) and fed to the GEMM; the result is
    compared with the oracle run on the oracle's own quantization, and with the unquantized fp32 linear."""
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    K, N = 7168, 2048
    x = make_activation(M, K)
    w_q, w_s = make_fp8_weight(N, K)
    x_q, x_s = per_token_group_quant_fp8(x.to(gpu), 128, column_major_scales=True)
    out = fp8_blockwise_scaled_mm(x_q, w_q.to(gpu).t(), x_s, w_s.to(gpu).t(), torch.bfloat16)
    q_o, s_o = oracle.group_quant(x, 128, mode="div", layout="col")
    assert torch.equal(x_q.cpu().view(torch.uint8), q_o.view(torch.uint8)) and torch.equal(x_s.cpu(), s_o)
    ref, mag = oracle.fp8_blockwise_mm(q_o, w_q, s_o, w_s, torch.float32, want_abs=True)
    _check(out, ref, mag, "single linear", FP8_MAG_TOL_CONFIG, 0.9975)
    assert tuple(out.shape) == (M, N) and bool(torch.isfinite(out).all())


def test_outlier_scales_do_not_overflow(gpu, oracle):
    """Huge activation outliers: large scales on the activation side, no NaN/Inf in bf16 output."""
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8, w8a8_block_fp8_matmul

    x = make_activation(64, 1024, seed=2, outlier_frac=0.01, outlier_gain=1e4)
    w_q, w_s = make_fp8_weight(512, 1024, seed=3)
    x_q, x_s = per_token_group_quant_fp8(x.to(gpu), 128)
    out = w8a8_block_fp8_matmul(x_q, w_q.to(gpu), x_s, w_s.to(gpu), [128, 128], torch.bfloat16)
    ref, mag = oracle.fp8_blockwise_mm(x_q.cpu(), w_q, x_s.cpu(), w_s, torch.float32, want_abs=True)
    _check(out, ref, mag, "outliers")


def test_full_size_prefill_shape_properties(gpu, oracle):
    """M=4096, K=7168 -> N=4608 (a DeepSeek-V3 shape of the reference's test list): too big for the oracle
    in full, so (1) a random sample of rows and columns is checked against the oracle, (2) linearity in the
    scales: doubling sa doubles the output exactly (powers of two commute with every rounding)."""
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul

    M, N, K = 4096, 4608, 7168
    g = torch.Generator().manual_seed(5)
    a = torch.randint(0, 256, (M, K), generator=g, dtype=torch.uint8)
    a = torch.where((a & 0x7F) == 0x7F, a & 0xF7, a).view(FP8)
    w = torch.randint(0, 256, (N, K), generator=g, dtype=torch.uint8)
    w = torch.where((w & 0x7F) == 0x7F, w & 0xF7, w).view(FP8)
    As = torch.rand(M, K // 128, generator=g) * 1e-3
    Bs = torch.rand(N // 128, K // 128, generator=g) * 1e-3
    ag, wg, Asg, Bsg = a.to(gpu), w.to(gpu), As.to(gpu), Bs.to(gpu)
    out = w8a8_block_fp8_matmul(ag, wg, Asg, Bsg, [128, 128], torch.bfloat16)
    rows = torch.randperm(M, generator=g)[:48]
    rows = torch.cat([rows, torch.tensor([0, 255, 256, M - 1])])
    ref, mag = oracle.fp8_blockwise_mm(a[rows].contiguous(), w, As[rows].contiguous(), Bs, torch.float32, want_abs=True)
    _check(out[rows.to(gpu)], ref, mag, "sampled rows")
    out2 = w8a8_block_fp8_matmul(ag, wg, Asg * 2, Bsg, [128, 128], torch.bfloat16)
    assert torch.equal(out2.float(), out.float() * 2)


# Large-M kernels: 256x256 direct-to-LDS tiles (>= 256 such tiles) and 256x128 pipelined tiles, each with K a multiple of
# 128 and not, and with ragged M and N edges.  The oracle checks a sample of rows (first, last, tile borders, random).
@pytest.mark.parametrize("M,N,K", [(4096, 4352, 512), (4000, 4300, 400), (4096, 2176, 512), (4096, 2176, 256), (4000, 2100, 272),
                                   (8192, 2048, 1024)])
def test_large_m_kernels(gpu, oracle, M, N, K):
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul

    print(f"case M={M} N={N} K={K}", flush=True)
    g = torch.Generator().manual_seed(M + N + K)
    a, w = _rand_fp8((M, K), g), _rand_fp8((N, K), g)
    As = torch.rand(M, cdiv(K, 128), generator=g) * 1e-2
    Bs = torch.rand(cdiv(N, 128), cdiv(K, 128), generator=g) * 1e-2
    out = w8a8_block_fp8_matmul(a.to(gpu), w.to(gpu), As.to(gpu), Bs.to(gpu), [128, 128], torch.bfloat16)
    rows = torch.cat([torch.tensor([0, 1, 127, 128, 255, 256, 257, M - 257, M - 256, M - 2, M - 1]),
                      torch.randperm(M, generator=g)[:40]])
    ref, mag = oracle.fp8_blockwise_mm(a[rows].contiguous(), w, As[rows].contiguous(), Bs, torch.float32, want_abs=True)
    _check(out[rows.to(gpu)], ref, mag, f"M={M} N={N} K={K}")
    assert bool(torch.isfinite(out).all())
