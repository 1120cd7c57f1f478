"""GPU parity of the per-token x per-channel INT8 GEMM and of the per-token INT8 quantizer.

Integer work is held to bit-exactness: the int32 accumulators (read back through the raw-accumulator
hook of the C ABI) must equal exact integer arithmetic, and the bf16/fp16 output must equal the oracle's
epilogue f32(acc) * (sb[n] * sa[m]) + bias bit for bit.  Against the reference's other two epilogue
orders (which differ in fp32 rounding only) at most one unit in the last place is allowed, and the
reference's own test criterion (assert_close defaults against the fp32 torch formula) must hold.
"""
import pytest
import torch

from sglang_amd.workloads import make_int8_activation, make_int8_weight

pytestmark = pytest.mark.gpu

SHAPES = [
    (1, 16, 512), (1, 6144, 4096), (16, 128, 512), (17, 136, 1024), (32, 512, 4096), (64, 1024, 512),
    (100, 4096, 1024), (128, 16384, 512), (256, 6144, 4096), (300, 4096, 14336), (512, 264, 16384),
    (1024, 512, 1024), (1, 4096, 14336), (4, 28672, 512),
]


def _bits16(t):
    return t.cpu().view(torch.int16).to(torch.int32)


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_int32_accumulators_are_exact(gpu, oracle, M, N, K):
    from sglang_amd import ops

    print(f"case M={M} N={N} K={K}", flush=True)
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    acc = ops.int8_mm_raw_accumulators(a.to(gpu), w.to(gpu).t())
    assert acc.dtype == torch.int32
    want = oracle.int8_mm_acc(a, w)
    assert torch.equal(acc.cpu(), want)


def test_int32_accumulator_extremes(gpu):
    from sglang_amd import ops

    K = 14336
    a = torch.full((3, K), -128, dtype=torch.int8)
    w = torch.full((16, K), -128, dtype=torch.int8)
    w[1] = 127
    acc = ops.int8_mm_raw_accumulators(a.to(gpu), w.to(gpu).t()).cpu()
    assert acc[0, 0] == 128 * 128 * K and acc[2, 1] == -128 * 127 * K


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_int8_scaled_mm(gpu, oracle, M, N, K, with_bias, out_dtype):
    from sglang_amd.sgl_kernel import int8_scaled_mm

    print(f"case M={M} N={N} K={K} bias={with_bias} {out_dtype}", flush=True)
    a, sa = make_int8_activation(M, K)
    w, sb = make_int8_weight(N, K)
    g = torch.Generator().manual_seed(N)
    bias = (torch.randn(N, generator=g) * 10).to(out_dtype) if with_bias else None
    out = int8_scaled_mm(a.to(gpu), w.to(gpu).t(), sa.to(gpu), sb.to(gpu), out_dtype,
                         bias.to(gpu) if with_bias else None)
    assert out.dtype == out_dtype and tuple(out.shape) == (M, N)
    acc = oracle.int8_mm_acc(a, w)
    want = oracle.int8_epilogue(acc, sa, sb, out_dtype, bias, oracle.EPI_COL_ROW)
    assert torch.equal(_bits16(out), _bits16(want))
    if not with_bias:  # (a bias that nearly cancels the product turns one fp32 ulp into several output ulps)
        for order in (oracle.EPI_ROW_COL_ACC, oracle.EPI_TORCH):
            other = oracle.int8_epilogue(acc, sa, sb, out_dtype, None, order)
            assert int((_bits16(out) - _bits16(other)).abs().max()) <= 1
    # the reference's own test: torch fp32 formula, assert_close defaults
    o = acc.float() * sa.view(-1, 1) * sb.view(1, -1)
    if with_bias:
        o = o + bias
    torch.testing.assert_close(out.cpu(), o.to(out_dtype))


@pytest.mark.parametrize("M,N,K", [(4096, 4096, 512), (4000, 4088, 1024), (2048, 8192, 256)])
def test_large_m_kernel(gpu, oracle, M, N, K):
    """The 256x256 direct-to-LDS kernel (16x16x64 MFMA): raw accumulators and epilogue on a sample of rows that includes
    tile borders and the ragged last tile, all columns."""
    from sglang_amd import ops
    from sglang_amd.sgl_kernel import int8_scaled_mm

    print(f"case M={M} N={N} K={K}", flush=True)
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    sa, sb = torch.rand(M, generator=g) * 0.1, torch.rand(N, generator=g) * 0.01
    bias = (torch.randn(N, generator=g) * 10).to(torch.bfloat16)
    ag, wg = a.to(gpu), w.to(gpu)
    acc = ops.int8_mm_raw_accumulators(ag, wg.t())
    out = int8_scaled_mm(ag, wg.t(), sa.to(gpu), sb.to(gpu), torch.bfloat16, bias.to(gpu))
    rows = torch.cat([torch.tensor([0, 31, 32, 127, 128, 255, 256, M - 257, M - 33, M - 2, M - 1]),
                      torch.randperm(M, generator=g)[:24]])
    want_acc = oracle.int8_mm_acc(a[rows].contiguous(), w)
    assert torch.equal(acc[rows.to(gpu)].cpu(), want_acc)
    want = oracle.int8_epilogue(want_acc, sa[rows], sb, torch.bfloat16, bias)
    assert torch.equal(_bits16(out[rows.to(gpu)]), _bits16(want))


def test_reference_test_distribution(gpu, oracle):
    """sgl-kernel/tests/test_int8_gemm.py:20-31: int8 from randn*5, scales randn (negative values included)."""
    from sglang_amd.sgl_kernel import int8_scaled_mm

    g = torch.Generator().manual_seed(0)
    M, N, K = 64, 1024, 4096
    a = torch.round((torch.randn(M, K, generator=g) * 5).clamp(-128, 127)).to(torch.int8)
    w = torch.round((torch.randn(N, K, generator=g) * 5).clamp(-128, 127)).to(torch.int8)
    sa, sb = torch.randn(M, generator=g), torch.randn(N, generator=g)
    bias = (torch.randn(N, generator=g) * 10).to(torch.bfloat16)
    out = int8_scaled_mm(a.to(gpu), w.to(gpu).t(), sa.to(gpu), sb.to(gpu), torch.bfloat16, bias.to(gpu))
    want = oracle.int8_scaled_mm(a, w, sa, sb, torch.bfloat16, bias)
    assert torch.equal(_bits16(out), _bits16(want))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M,K", [(1, 512), (7, 4096), (64, 14336), (33, 16384 + 512), (5, 8192), (6, 2056), (9, 8200)])
def test_per_token_quant_int8(gpu, oracle, dtype, M, K):
    from sglang_amd.int8_kernel import per_token_quant_int8
    from sglang_amd.workloads import make_activation

    x = make_activation(M, K, seed=M + K, dtype=dtype)
    q, s = per_token_quant_int8(x.to(gpu))
    q_o, s_o = oracle.per_token_quant_int8(x)
    assert q.dtype == torch.int8 and tuple(s.shape) == (M, 1)
    assert torch.equal(s.cpu().view(torch.int32), s_o.view(torch.int32))
    assert torch.equal(q.cpu(), q_o)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M,K", [(1, 512), (7, 4096), (64, 14336), (33, 16384 + 512), (6, 2056)])
def test_per_token_quant_int8_with_row_sums(gpu, oracle, dtype, M, K):
    """per_token_quant_int8(cal_sum=True), int8_kernel.py:52-54, :66-69: codes and scales unchanged (bit for bit), plus the
    row sums in the input's type.  The reference's fp32 reduction order is Triton's, not defined by the source, so the sum is
    held to the exact (fp64) sum within fp32 reassociation error, K * 2^-24 * sum|x|, plus half a unit of the output type;
    a row of small integers, where every partial sum is exact, must come back exactly."""
    from sglang_amd.int8_kernel import per_token_quant_int8
    from sglang_amd.workloads import make_activation

    x = make_activation(M, K, seed=M + K, dtype=dtype)
    x[0] = torch.randint(-3, 4, (K,), generator=torch.Generator().manual_seed(K)).to(dtype)
    q, s, x_sum = per_token_quant_int8(x.view(1, M, K).to(gpu), cal_sum=True)
    assert x_sum.dtype == dtype and tuple(x_sum.shape) == (1, M) and tuple(s.shape) == (1, M, 1) and q.dtype == torch.int8
    q_o, s_o = oracle.per_token_quant_int8(x)
    assert torch.equal(s.cpu().view(M, 1).view(torch.int32), s_o.view(torch.int32)) and torch.equal(q.cpu().view(M, K), q_o)
    exact, mag, rounded = oracle.per_token_row_sum(x)
    got = x_sum.cpu().view(M).double()
    half_ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -24}[dtype]
    assert bool(((got - exact).abs() <= half_ulp * 1.001 * exact.abs() + K * 2.0 ** -24 * mag + 1e-30).all())
    assert got[0] == exact[0] == float(rounded[0])


def test_int8_linear_end_to_end(gpu, oracle):
    """W8A8Int8LinearMethod.apply (python/sglang/srt/layers/quantization/w8a8_int8.py:387-417):
    per_token_quant_int8 then int8_scaled_mm, against the bf16 linear it approximates."""
    from sglang_amd.int8_kernel import per_token_quant_int8
    from sglang_amd.sgl_kernel import int8_scaled_mm
    from sglang_amd.workloads import make_activation

    M, K, N = 48, 4096, 6144
    x = make_activation(M, K, seed=9, outlier_frac=0.0)
    w_q, w_s = make_int8_weight(N, K)
    x_q, x_s = per_token_quant_int8(x.to(gpu))
    out = int8_scaled_mm(x_q, w_q.to(gpu).t(), x_s, w_s.to(gpu), torch.bfloat16)
    ref = x.float() @ (w_q.float() * w_s[:, None]).T
    rel = (out.float().cpu() - ref).norm() / ref.norm()
    assert float(rel) < 0.02
