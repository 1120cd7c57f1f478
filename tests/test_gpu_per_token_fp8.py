"""GPU parity of the per-token x per-channel FP8 linear: sgl_per_token_quant_fp8 (codes and scales bit-exact) and
fp8_scaled_mm (floating point: |out - ref| <= 1e-2 * |ref| + 1e-4 * mag, mag = |sa * sb| * sum |a * b|, the slack the
grouped additions of the fp8 MFMA need where large terms cancel, see tests/test_gpu_fp8_gemm.py; plus the reference's own
criterion rtol 0.02 / atol 1 against its torch formula, sgl-kernel/tests/test_fp8_gemm.py:7-37)."""
import pytest
import torch

from fp8_tolerance import check_fp8_gemm
from sglang_amd.workloads import make_activation

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M,K", [(1, 512), (7, 4096), (64, 7168), (33, 16384 + 512), (3, 8), (5, 8192), (6, 2056), (9, 8200)])
def test_per_token_quant_fp8_bits(gpu, oracle, dtype, M, K):
    from sglang_amd.fp8_kernel import sglang_per_token_quant_fp8

    if dtype == torch.float32 and K % 4:
        pytest.skip("row must span a multiple of 16 bytes")
    x = make_activation(M, K, seed=M * 7 + K, dtype=dtype)
    if M > 2:
        x[1] = 0  # a row of zeros: scale 0, codes 0, no NaN
    q, s = sglang_per_token_quant_fp8(x.to(gpu))
    q_o, s_o = oracle.per_token_quant_fp8(x)
    assert q.dtype == FP8 and tuple(s.shape) == (M, 1)
    assert torch.equal(s.cpu().view(torch.int32), s_o.view(torch.int32))
    assert torch.equal(q.cpu().view(torch.uint8), q_o.view(torch.uint8))
    if M > 2:
        assert float(s[1]) == 0.0 and not bool(q[1].view(torch.uint8).any())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M,K", [(3, 7168), (130, 4096), (5, 2056), (2, 18432), (7, 1536)])
@pytest.mark.parametrize("column_major", [False, True])
def test_whole_row_group_quant_bits(gpu, oracle, dtype, M, K, column_major):
    """per_token_group_quant_fp8 with group_size == K (a weight quantized per output channel at load time): rows longer than
    the group kernel's groups, not powers of two; row-major scales multiply by the reciprocal, column-major ones divide."""
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8

    x = make_activation(M, K, seed=M * 11 + K, dtype=dtype)
    x[1] = 0  # a row of zeros: the floor eps keeps the scale positive, codes are zero
    q, s = per_token_group_quant_fp8(x.to(gpu), K, column_major_scales=column_major)
    q_o, s_o = oracle.group_quant(x, K, mode="div" if column_major else "rcp", layout="col" if column_major else "row")
    assert q.dtype == FP8 and tuple(s.shape) == (M, 1)
    assert torch.equal(s.cpu().contiguous().view(torch.int32), s_o.contiguous().view(torch.int32))
    assert torch.equal(q.cpu().view(torch.uint8), q_o.view(torch.uint8))
    assert float(s[1]) == pytest.approx(1e-10 / 448.0) and not bool(q[1].view(torch.uint8).any())


def _rand_fp8(shape, g):
    return ((torch.rand(*shape, generator=g) - 0.5) * 2 * 448.0).clamp(-448, 448).to(FP8)


# decode, mid-M (64- and 128-token tiles, split and whole), generic (ragged N), two-phase large-M
# (+ 192-channel tiles of the mid-M kernel, whole-K and split: the channel-scale epilogue follows their interleaved tiles)
SHAPES = [(1, 512, 1024), (16, 2048, 7168), (48, 16384, 2048), (130, 8192, 7168), (300, 1088, 512), (128, 16, 512),
          (1024, 1024, 4096), (4096, 4352, 512), (4000, 576, 1024), (100, 36864, 512), (130, 3072, 7168),
          (3990, 4304, 512),  # two-phase kernel with a ragged last token tile (6 of 16 rows) and a ragged last channel tile
          (8, 36864, 5760), (13, 24576, 1536)]  # decode sizes on one round of unsplit mid-M tiles (the token scales are re-laid out first)


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_fp8_scaled_mm(gpu, oracle, M, N, K, with_bias, out_dtype):
    from sglang_amd import _lib
    from sglang_amd.sgl_kernel import fp8_scaled_mm

    print(f"case M={M} N={N} K={K} bias={with_bias} {out_dtype} -> {_lib.gemm_plan('fp8', M, N, K)['kernel']}", flush=True)
    g = torch.Generator().manual_seed(M + 3 * N + K)
    a, w = _rand_fp8((M, K), g), _rand_fp8((N, K), g)
    sa = torch.randn(M, generator=g) * 1e-3
    sb = torch.randn(N, generator=g) * 1e-3
    bias = torch.randn(N, generator=g).to(out_dtype) if with_bias else None
    out = fp8_scaled_mm(a.to(gpu), w.to(gpu).t(), sa.to(gpu), sb.to(gpu), out_dtype, bias.to(gpu) if with_bias else None)
    assert out.dtype == out_dtype and tuple(out.shape) == (M, N)
    rows = torch.arange(M) if M <= 512 else torch.cat([torch.tensor([0, 255, 256, M - 1]), torch.randperm(M, generator=g)[:44]])
    ref, mag = oracle.fp8_scaled_mm(a[rows].contiguous(), w, sa[rows], sb, torch.float32, None, want_abs=True)
    if with_bias:
        ref = ref + bias.float()[None, :]
    # fp16 only: one step of the subnormal grid, the products of two 1e-3 scales reach down there
    check_fp8_gemm(out[rows.to(gpu)], ref, mag, f"M={M} N={N} K={K}", extra=2.0 ** -24 if out_dtype == torch.float16 else 0.0)
    # the reference's own test: torch formula, bias added after the cast
    o = (a[rows].float() @ w.float().T) * sa[rows].view(-1, 1) * sb.view(1, -1)
    o = o.to(out_dtype)
    if with_bias:
        o = o + bias.view(1, -1)
    torch.testing.assert_close(out[rows.to(gpu)].cpu(), o, rtol=0.02, atol=1.0)


def test_fp8_scaled_mm_exact_integers(gpu):
    """Integer codes and power-of-two scales: every product, sum and scaling is exact, whatever the order."""
    from sglang_amd.sgl_kernel import fp8_scaled_mm

    g = torch.Generator().manual_seed(6)
    for M, N, K in [(9, 384, 640), (300, 256, 1152), (2048, 4096, 256)]:
        ai = torch.randint(-8, 9, (M, K), generator=g)
        wi = torch.randint(-8, 9, (N, K), generator=g)
        sa = torch.exp2(torch.randint(-3, 4, (M,), generator=g).float())
        sb = torch.exp2(torch.randint(-3, 4, (N,), generator=g).float())
        bias = torch.randint(-16, 17, (N,), generator=g).float().to(torch.bfloat16)
        out = fp8_scaled_mm(ai.float().to(FP8).to(gpu), wi.float().to(FP8).to(gpu).t(), sa.to(gpu), sb.to(gpu), torch.bfloat16,
                            bias.to(gpu))
        want = ((ai.double() @ wi.double().T) * sa.double()[:, None] * sb.double()[None, :] + bias.double()[None, :])
        assert torch.equal(out.cpu().double(), want.to(torch.bfloat16).double()), (M, N, K)


@pytest.mark.parametrize("shape,N,K", [((2, 5), 384, 512), ((1,), 6144, 4096), ((700,), 1024, 2048), ((4096,), 1024, 1024),
                                       ((16,), 18432, 7168), ((5,), 264, 400)])
def test_apply_fp8_linear(gpu, oracle, shape, N, K):
    """apply_fp8_linear: per-token quantization then fp8_scaled_mm (one C-ABI call for both), against the oracle's pipeline,
    the unquantized linear, and the two operators called one after the other (bit for bit)."""
    from sglang_amd.fp8_kernel import sglang_per_token_quant_fp8
    from sglang_amd.fp8_utils import apply_fp8_linear
    from sglang_amd.sgl_kernel import fp8_scaled_mm

    M = 1
    for d in shape:
        M *= d
    x = make_activation(M, K, seed=5, outlier_frac=0.0).view(*shape, K)
    g = torch.Generator().manual_seed(8)
    w = torch.randn(N, K, generator=g) * 0.02
    w_s = w.abs().amax(1) / 448.0
    w_q = (w / w_s[:, None]).clamp(-448, 448).to(FP8)
    bias = torch.randn(N, generator=g).to(torch.bfloat16)
    out = apply_fp8_linear(x.to(gpu), w_q.to(gpu).t(), w_s.to(gpu), bias=bias.to(gpu))
    assert tuple(out.shape) == (*shape, N) and out.dtype == torch.bfloat16
    xq, xs = oracle.per_token_quant_fp8(x.view(M, K))
    ref, mag = oracle.fp8_scaled_mm(xq, w_q, xs, w_s, torch.float32, None, want_abs=True)
    ref = ref + bias.float()[None, :]
    check_fp8_gemm(out.view(M, N), ref, mag, "apply_fp8_linear")
    full = x.view(M, K).float() @ w.T + bias.float()
    assert float((out.float().cpu().view(M, N) - full).norm() / full.norm()) < 0.05
    q, s = sglang_per_token_quant_fp8(x.to(gpu).view(M, K))
    two = fp8_scaled_mm(q, w_q.to(gpu).t(), s, w_s.to(gpu), torch.bfloat16, bias.to(gpu))
    assert torch.equal(out.view(M, N).view(torch.int16), two.view(torch.int16))
