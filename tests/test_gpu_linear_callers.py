"""The linear-method callers (quantize -> GEMM -> bias -> reshape) against the same pipeline run on the CPU oracle."""
import pytest
import torch

from sglang_amd.workloads import make_activation, make_fp8_weight, make_int8_weight

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,N,K", [((2, 5), 384, 512), ((16,), 2048, 7168), ((3, 7), 576, 1024), ((300,), 1088, 384),
                                       ((1,), 7168, 2048), ((4100,), 1024, 256)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_block_fp8_linear(gpu, oracle, shape, N, K, with_bias):
    """One-call block-FP8 linear (quantize into the workspace, GEMM, bias in the epilogue) against the same pipeline on
    the oracle: q = x / s activation codes, blockwise GEMM in fp32, bias added in fp32, one rounding to bf16."""
    from sglang_amd import fp8_utils

    M = 1
    for d in shape:
        M *= d
    x = make_activation(M, K, seed=N + K).view(*shape, K)
    w_q, w_s = make_fp8_weight(N, K)
    g = torch.Generator().manual_seed(1)
    bias = torch.randn(N, generator=g).to(torch.bfloat16) if with_bias else None
    assert fp8_utils.dispatch_w8a8_block_fp8_linear() is fp8_utils.w8a8_block_fp8_linear
    for fn in (fp8_utils.cutlass_w8a8_block_fp8_linear_with_fallback, fp8_utils.triton_w8a8_block_fp8_linear):
        out = fn(x.to(gpu), w_q.to(gpu), [128, 128], w_s.to(gpu), None, bias.to(gpu) if with_bias else None)
        assert out.dtype == torch.bfloat16 and tuple(out.shape) == (*shape, N)
        xq, xs = oracle.group_quant(x.view(M, K), 128, mode="div")
        ref, mag = oracle.fp8_blockwise_mm(xq, w_q, xs, w_s, torch.float32, want_abs=True)
        want = ref + bias.float()[None, :] if with_bias else ref
        err = (out.float().cpu().view(M, N) - want).abs()
        tol = 1e-2 * want.abs() + 1e-4 * mag + (2.0 ** -8 * bias.float().abs()[None, :] if with_bias else 0)
        assert bool((err <= tol).all()), float((err - tol).max())
        assert bool(torch.isfinite(out).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(1, 2048, 7168), (3, 16640, 4480), (8, 7168, 18432), (16, 512, 512), (5, 66048, 512), (9, 256, 128)])
def test_decode_linear_quantizes_in_the_gemm_kernel(gpu, oracle, M, N, K, dtype):
    """At decode sizes the one-call linear has no quantizer launch: the GEMM kernel quantizes the tokens of each K range
    in its prologue.  Same arithmetic on the same codes and scales as quantizer + GEMM in two steps, so the outputs must
    be identical bit for bit (split and unsplit plans, several channel groups per workgroup, a short last K range, rows
    past M); the two-step path is held to the oracle elsewhere, and once more here."""
    from sglang_amd import _lib
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8
    from sglang_amd.fp8_utils import w8a8_block_fp8_linear
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    assert _lib.gemm_plan("fp8", M, N, K)["kernel"] == "decode"
    x = make_activation(M, K, seed=M + N, dtype=dtype)
    x[0, :128] = 0  # a group of zeros: scale 1e-10 / 448, codes 0
    w_q, w_s = make_fp8_weight(N, K, seed=K)
    xg, wg, sg = x.to(gpu), w_q.to(gpu), w_s.to(gpu)
    fused = w8a8_block_fp8_linear(xg, wg, [128, 128], sg)
    q, s = per_token_group_quant_fp8(xg, 128, column_major_scales=True)
    two_step = fp8_blockwise_scaled_mm(q, wg.t(), s, sg.t(), dtype)
    assert fused.dtype == dtype and torch.equal(fused.view(torch.int16), two_step.view(torch.int16))
    xq, xs = oracle.group_quant(x, 128, mode="div")
    ref, mag = oracle.fp8_blockwise_mm(xq, w_q, xs, w_s, torch.float32, want_abs=True)
    assert bool(((fused.float().cpu() - ref).abs() <= 1e-2 * ref.abs() + 1e-4 * mag).all())


def test_block_fp8_linear_ragged_k_falls_back(gpu, oracle):
    """K not a multiple of 128 cannot be group-quantized; N ragged is fine."""
    from sglang_amd.fp8_utils import w8a8_block_fp8_linear

    x = make_activation(8, 512, seed=3)
    w_q, w_s = make_fp8_weight(200, 512)
    out = w8a8_block_fp8_linear(x.to(gpu), w_q.to(gpu), [128, 128], w_s.to(gpu))
    xq, xs = oracle.group_quant(x, 128, mode="div")
    ref, mag = oracle.fp8_blockwise_mm(xq, w_q, xs, w_s, torch.float32, want_abs=True)
    assert bool(((out.float().cpu() - ref).abs() <= 1e-2 * ref.abs() + 1e-4 * mag).all())
    with pytest.raises(NotImplementedError):
        w8a8_block_fp8_linear(x.to(gpu), w_q.to(gpu), [64, 64], w_s.to(gpu))


@pytest.mark.parametrize("shape,N,K", [((4, 3), 6144, 4096), ((1,), 4096, 14336), ((300,), 264, 512)])
def test_int8_linear(gpu, oracle, shape, N, K):
    from sglang_amd.w8a8_int8 import apply_w8a8_int8_linear

    M = 1
    for d in shape:
        M *= d
    x = make_activation(M, K, seed=N, outlier_frac=0.0).view(*shape, K)
    w_q, w_s = make_int8_weight(N, K)
    g = torch.Generator().manual_seed(2)
    bias = torch.randn(N, generator=g).to(torch.bfloat16)
    out = apply_w8a8_int8_linear(x.to(gpu), w_q.to(gpu).t(), w_s.view(N, 1).to(gpu), bias.to(gpu))
    assert tuple(out.shape) == (*shape, N) and out.dtype == torch.bfloat16
    xq, xs = oracle.per_token_quant_int8(x.view(M, K))
    want = oracle.int8_scaled_mm(xq, w_q, xs, w_s, torch.bfloat16, bias)
    assert torch.equal(out.cpu().view(M, N).view(torch.int16), want.view(torch.int16))
