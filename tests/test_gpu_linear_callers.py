"""The linear-method callers (quantize -> GEMM -> bias -> reshape) against the same pipeline run on the CPU oracle."""
import pytest
import torch

from sglang_amd.workloads import make_activation, make_fp8_weight, make_int8_weight
from test_gpu_fp8_gemm import FP8_MAG_TOL

pytestmark = pytest.mark.gpu


def _bias_after_rounding(out_nobias: torch.Tensor, bias: torch.Tensor, oracle) -> torch.Tensor:
    """`output += bias` of fp8_utils.py:208-209 / :296-297 on the CPU: both operands are 16-bit, the sum is formed in
    fp32 and rounded to the 16-bit type again (the oracle's rounding routines, pinned against torch's casts)."""
    s = out_nobias.float().cpu() + bias.float().cpu()[None, :]
    if out_nobias.dtype == torch.bfloat16:
        return oracle.f32_to_bf16_bits(s)
    return oracle.f32_to_f16_bits(s)


@pytest.mark.parametrize("shape,N,K", [((2, 5), 384, 512), ((16,), 2048, 7168), ((3, 7), 576, 1024), ((300,), 1088, 384),
                                       ((1,), 7168, 2048), ((4100,), 1024, 256), ((40,), 200, 384),
                                       # decode sizes where the wrappers' one call quantizes inside the GEMM kernel: producer
                                       # waves of the mid-M kernel, the streaming kernel's prologue (split, with a short last range)
                                       ((13,), 53248, 1152), ((2, 4), 24576, 1536), ((14,), 16640, 4480), ((8,), 36800, 1280),
                                       ((2,), 36864, 5760), ((1,), 28672, 4096)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_block_fp8_linear_wrappers_follow_the_reference(gpu, oracle, shape, N, K, dtype):
    """The two block-FP8 wrappers of the reference are different computations (fp8_utils.py:184-214 vs :281-301):
    the CUTLASS one quantizes with `x / s` and M-major scales and calls `fp8_blockwise_scaled_mm`, the Triton one
    quantizes with `x * (1 / s)` and row-major scales and calls `w8a8_block_fp8_matmul`; the first falls back to the
    second when N or K is not a multiple of 128; both add the bias to the already rounded output.  Checked here:
    (1) the activation codes and scales each wrapper's quantizer call produces are the oracle's for that rounding mode,
    bit for bit; (2) each wrapper's output without bias is within the GEMM tolerance of the oracle's product of the oracle's
    codes, and equals its two-step sequence through the operator entry points bit for bit wherever the wrapper's one call
    multiplies with the kernel the GEMM entry point takes (everywhere but at some decode shapes, where it takes a kernel that
    quantizes the tokens itself and adds the same products in another order); (3) with a bias the
    output equals round(round(GEMM) + bias) bit for bit - the reference's order, computed on the CPU."""
    from sglang_amd import fp8_utils
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8, w8a8_block_fp8_matmul
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm
    from test_gpu_fp8_gemm import _check

    M = 1
    for d in shape:
        M *= d
    ragged = N % 128 != 0  # K % 128 == 0 always: the 1x128 quantizer of either wrapper asserts it, as the reference's does
    x = make_activation(M, K, seed=N + K, dtype=dtype).view(*shape, K)
    w_q, w_s = make_fp8_weight(N, K)
    g = torch.Generator().manual_seed(1)
    bias = torch.randn(N, generator=g).to(dtype)
    xg, wg, sg, bg = x.to(gpu), w_q.to(gpu), w_s.to(gpu), bias.to(gpu)
    assert fp8_utils.dispatch_w8a8_block_fp8_linear() is fp8_utils.cutlass_w8a8_block_fp8_linear_with_fallback
    assert fp8_utils.cutlass_w8a8_block_fp8_linear_with_fallback is not fp8_utils.triton_w8a8_block_fp8_linear

    for fn, mode in ((fp8_utils.cutlass_w8a8_block_fp8_linear_with_fallback, "rcp" if ragged else "div"),
                     (fp8_utils.triton_w8a8_block_fp8_linear, "rcp")):
        col = mode == "div"
        q, s = per_token_group_quant_fp8(xg.view(M, K), 128, column_major_scales=col)
        q_o, s_o = oracle.group_quant(x.view(M, K), 128, mode=mode, layout="col" if col else "row")
        assert torch.equal(q.cpu().view(torch.uint8), q_o.view(torch.uint8)) and torch.equal(s.cpu(), s_o)
        if col:
            two_step = fp8_blockwise_scaled_mm(q, wg.t(), s, sg.t(), dtype)
        else:
            two_step = w8a8_block_fp8_matmul(q, wg, s, sg, [128, 128], output_dtype=dtype)
        plain = fn(xg, wg, [128, 128], sg, None, None)
        assert plain.dtype == dtype and tuple(plain.shape) == (*shape, N)
        ref, mag = oracle.fp8_blockwise_mm(q_o, w_q, s_o, w_s, torch.float32, want_abs=True)
        _check(plain.reshape(M, N), ref, mag, f"{fn.__name__} M={M} N={N} K={K}")
        if fp8_utils._one_call_takes_the_same_gemm(M, N, K):
            assert torch.equal(plain.reshape(M, N).view(torch.int16), two_step.view(torch.int16))
        else:  # the one call takes a kernel that quantizes the tokens itself, the GEMM entry point another: other order of sums
            _check(two_step, ref, mag, f"two calls M={M} N={N} K={K}")
        biased = fn(xg, wg, [128, 128], sg, None, bg)
        want = _bias_after_rounding(plain.reshape(M, N), bias, oracle)
        assert torch.equal(biased.reshape(M, N).cpu().view(torch.int16), want.view(torch.int16))
        assert bool(torch.isfinite(biased).all())


def test_the_two_wrappers_round_activations_differently(gpu, oracle):
    """`x / s` and `x * (1 / s)` disagree on a fraction of a percent of the codes (never on the scales); the wrappers
    must reproduce that difference, not share one quantizer."""
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8

    x = make_activation(512, 2048, seed=77)
    q_div, s_div = oracle.group_quant(x, 128, mode="div")
    q_rcp, s_rcp = oracle.group_quant(x, 128, mode="rcp")
    differ = int((q_div.view(torch.uint8) != q_rcp.view(torch.uint8)).sum())
    assert torch.equal(s_div, s_rcp) and 0 < differ < 0.005 * x.numel()
    q_c, _ = per_token_group_quant_fp8(x.to(gpu), 128, column_major_scales=True)
    q_t, _ = per_token_group_quant_fp8(x.to(gpu), 128, column_major_scales=False)
    assert torch.equal(q_c.cpu().view(torch.uint8), q_div.view(torch.uint8))
    assert torch.equal(q_t.cpu().view(torch.uint8), q_rcp.view(torch.uint8))


@pytest.mark.parametrize("shape,N,K", [((2, 5), 384, 512), ((16,), 2048, 7168), ((300,), 1152, 384), ((1,), 7168, 2048),
                                       ((4100,), 1024, 256)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_fused_block_fp8_linear(gpu, oracle, shape, N, K, with_bias):
    """This library's one-call linear (an opt-in with no counterpart in the reference): without a bias bit-identical to
    the CUTLASS-style wrapper; with one, the bias is added in fp32 before the single rounding, which is held against the
    oracle pipeline in that order and differs from the wrapper's twice-rounded output by at most the two roundings the
    wrapper makes (of the product, then of the sum)."""
    from sglang_amd import fp8_utils

    M = 1
    for d in shape:
        M *= d
    x = make_activation(M, K, seed=N + K).view(*shape, K)
    w_q, w_s = make_fp8_weight(N, K)
    g = torch.Generator().manual_seed(1)
    bias = torch.randn(N, generator=g).to(torch.bfloat16) if with_bias else None
    xg, wg, sg = x.to(gpu), w_q.to(gpu), w_s.to(gpu)
    out = fp8_utils.fused_w8a8_block_fp8_linear(xg, wg, [128, 128], sg, None, bias.to(gpu) if with_bias else None)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (*shape, N)
    two = fp8_utils.cutlass_w8a8_block_fp8_linear_with_fallback(xg, wg, [128, 128], sg, None, bias.to(gpu) if with_bias else None)
    if not with_bias:
        assert torch.equal(out.view(torch.int16), two.view(torch.int16))
    else:
        # the wrapper rounds the product (half a unit of ITS last place, up to 2^-8 of it) and then the sum
        plain = fp8_utils.cutlass_w8a8_block_fp8_linear_with_fallback(xg, wg, [128, 128], sg).float()
        a, b = out.float(), two.float()
        within = (a - b).abs() <= 2.0 ** -8 * 1.01 * (plain.abs() + a.abs() + b.abs())  # three roundings, half a unit each
        assert bool(within.all()), int((~within).sum())
    xq, xs = oracle.group_quant(x.view(M, K), 128, mode="div")
    ref, mag = oracle.fp8_blockwise_mm(xq, w_q, xs, w_s, torch.float32, want_abs=True)
    want = ref + bias.float()[None, :] if with_bias else ref
    err = (out.float().cpu().view(M, N) - want).abs()
    tol = 1e-2 * want.abs() + FP8_MAG_TOL * mag
    assert bool((err <= tol).all()), float((err - tol).max())
    assert bool(torch.isfinite(out).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(1, 2048, 7168), (12, 2048, 7168), (14, 16640, 4480), (8, 4096, 18432), (16, 512, 512), (5, 66048, 512),
                                   (9, 256, 128), (4, 7168, 18432), (16, 7168, 2048),
                                   (16, 24576, 1536), (5, 36864, 5760), (13, 53248, 1152), (16, 32768, 1152), (13, 45056, 1280),
                                   (2, 36864, 5760), (3, 24576, 5120), (8, 36800, 5760)])
def test_decode_linear_quantizes_in_the_gemm_kernel(gpu, oracle, M, N, K, dtype):
    """At decode sizes the one-call linear has no quantizer launch: the streaming decode kernel quantizes the tokens of
    each K range in its prologue.  Same arithmetic on the same codes and scales as quantizer + GEMM in two steps, so where
    the two-step GEMM takes the same kernel the outputs must be identical bit for bit (split and unsplit plans, several
    channel groups per workgroup, a short last K range, rows past M).  Where the two-step GEMM takes the wave-split decode
    kernel instead (M = 1 here) the sums are added in another order and both are held to the oracle.  The last two shapes
    (K of 144 blocks; K of 16 blocks with 16 tokens) are ones where the one-call linear itself launches the quantizer and
    the wave-split kernel, being faster there: identical to the two steps again.  The five after them take the mid-M kernel on
    one round of unsplit 64-token tiles (128-, 192- and 256-channel tiles: six, four and three stages; K of 12, 45, 9, 9 and
    10 blocks), whose producer waves quantize the tokens: identical to quantizer + that kernel; the last two take it for the linear only
    (fewer tokens than the GEMM's own threshold; K of five ranges for the streaming kernel)."""
    from sglang_amd import _lib
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8
    from sglang_amd.fp8_utils import fused_w8a8_block_fp8_linear as w8a8_block_fp8_linear
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    kernel = _lib.gemm_plan("fp8", M, N, K)["kernel"]
    two_launches = (M, N, K) in ((4, 7168, 18432), (16, 7168, 2048))
    producer = (M, N, K) in ((16, 24576, 1536), (5, 36864, 5760), (13, 53248, 1152), (16, 32768, 1152), (13, 45056, 1280),
                            (8, 36800, 5760))  # (the last with a ragged last channel tile: 128 of 192 channels)
    linear_only = (M, N, K) in ((2, 36864, 5760), (3, 24576, 5120))  # the GEMM alone takes the wave-split kernel, the linear the producers
    assert kernel == ("dma3" if producer else "decode_wavesplit" if M == 1 or two_launches or linear_only else "decode")
    lin = _lib.block_linear_plan(M, N, K)
    assert (lin["quantizer"], lin["kernel"]) == (("fused", "dma3") if producer or linear_only else ("launch", "decode_wavesplit") if two_launches else ("fused", "decode"))
    x = make_activation(M, K, seed=M + N, dtype=dtype)
    x[0, :128] = 0  # a group of zeros: scale 1e-10 / 448, codes 0
    w_q, w_s = make_fp8_weight(N, K, seed=K)
    xg, wg, sg = x.to(gpu), w_q.to(gpu), w_s.to(gpu)
    fused = w8a8_block_fp8_linear(xg, wg, [128, 128], sg)
    q, s = per_token_group_quant_fp8(xg, 128, column_major_scales=True)
    if N % 128 == 0:
        two_step = fp8_blockwise_scaled_mm(q, wg.t(), s, sg.t(), dtype)
    else:  # the reference's operator refuses a ragged N (its scale-shape check); the Triton-style one takes it
        from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul

        two_step = w8a8_block_fp8_matmul(q, wg, s, sg, [128, 128], dtype)
    assert fused.dtype == dtype
    if kernel in ("decode", "dma3") or two_launches:
        assert torch.equal(fused.view(torch.int16), two_step.view(torch.int16))
    xq, xs = oracle.group_quant(x, 128, mode="div")
    ref, mag = oracle.fp8_blockwise_mm(xq, w_q, xs, w_s, torch.float32, want_abs=True)
    for out in (fused, two_step):
        assert bool(((out.float().cpu() - ref).abs() <= 1e-2 * ref.abs() + FP8_MAG_TOL * mag).all())


@pytest.mark.parametrize("M,N,K", [(16, 53248, 1280), (16, 53248, 1408), (16, 45056, 1408), (16, 32768, 1664), (16, 32768, 1792),
                                   (16, 32768, 2176)])
def test_producer_wave_linear_every_tail_length(gpu, M, N, K):
    """The producer waves and the other waves of the mid-M kernel must meet at the same number of barriers whatever is left of K
    after whole trips over the stages: three stages with 1 and 2 blocks left, four with 3, six with 1, 2 and 5 (0 and the other
    remainders are in the test above).  Bit-identical to quantizer + GEMM."""
    from sglang_amd import _lib
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8
    from sglang_amd.fp8_utils import fused_w8a8_block_fp8_linear
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    lin = _lib.block_linear_plan(M, N, K)
    assert (lin["kernel"], lin["quantizer"]) == ("dma3", "fused") and (K // 128) % lin["stages"] != 0
    print(f"case M={M} N={N} K={K}: {lin}", flush=True)
    x = make_activation(M, K, seed=N + K)
    w_q, w_s = make_fp8_weight(N, K, seed=K)
    xg, wg, sg = x.to(gpu), w_q.to(gpu), w_s.to(gpu)
    fused = fused_w8a8_block_fp8_linear(xg, wg, [128, 128], sg)
    q, s = per_token_group_quant_fp8(xg, 128, column_major_scales=True)
    two_step = fp8_blockwise_scaled_mm(q, wg.t(), s, sg.t(), torch.bfloat16)
    assert torch.equal(fused.view(torch.int16), two_step.view(torch.int16))


def test_block_fp8_linear_ragged_n_falls_back_to_the_triton_wrapper(gpu, oracle):
    """N not a multiple of 128: the CUTLASS-style wrapper hands over to the Triton-style one (fp8_utils.py:195-201),
    i.e. `x * (1 / s)` codes; K must be a multiple of the group size for either quantizer."""
    from sglang_amd.fp8_utils import cutlass_w8a8_block_fp8_linear_with_fallback, triton_w8a8_block_fp8_linear

    x = make_activation(8, 512, seed=3)
    w_q, w_s = make_fp8_weight(200, 512)
    out = cutlass_w8a8_block_fp8_linear_with_fallback(x.to(gpu), w_q.to(gpu), [128, 128], w_s.to(gpu))
    same = triton_w8a8_block_fp8_linear(x.to(gpu), w_q.to(gpu), [128, 128], w_s.to(gpu))
    assert torch.equal(out.view(torch.int16), same.view(torch.int16))
    xq, xs = oracle.group_quant(x, 128, mode="rcp")
    ref, mag = oracle.fp8_blockwise_mm(xq, w_q, xs, w_s, torch.float32, want_abs=True)
    assert bool(((out.float().cpu() - ref).abs() <= 1e-2 * ref.abs() + FP8_MAG_TOL * mag).all())


@pytest.mark.parametrize("shape,N,K", [((4, 3), 6144, 4096), ((1,), 4096, 14336), ((300,), 264, 512), ((256,), 4096, 14336),
                                       ((16,), 28672, 4096), ((2, 64), 6144, 4096), ((5,), 4096, 4112)])
@pytest.mark.parametrize("dtype,with_bias", [(torch.bfloat16, True), (torch.float16, False)])
def test_int8_linear(gpu, oracle, shape, N, K, dtype, with_bias):
    """The INT8 linear method's forward pass (w8a8_int8.py:387-417) is one C-ABI call: the oracle's codes, scales and
    product bit for bit (integer arithmetic and one rounding), hence also the two operators called one after the other."""
    from sglang_amd.int8_kernel import per_token_quant_int8
    from sglang_amd.sgl_kernel import int8_scaled_mm
    from sglang_amd.w8a8_int8 import apply_w8a8_int8_linear

    M = 1
    for d in shape:
        M *= d
    x = make_activation(M, K, seed=N, outlier_frac=0.0, dtype=dtype).view(*shape, K)
    w_q, w_s = make_int8_weight(N, K)
    g = torch.Generator().manual_seed(2)
    bias = torch.randn(N, generator=g).to(dtype) if with_bias else None
    xg, wg, sg, bg = x.to(gpu), w_q.to(gpu).t(), w_s.view(N, 1).to(gpu), bias.to(gpu) if with_bias else None
    out = apply_w8a8_int8_linear(xg, wg, sg, bg)
    assert tuple(out.shape) == (*shape, N) and out.dtype == dtype
    xq, xs = oracle.per_token_quant_int8(x.view(M, K))
    want = oracle.int8_scaled_mm(xq, w_q, xs, w_s, dtype, bias)
    assert torch.equal(out.cpu().view(M, N).view(torch.int16), want.view(torch.int16))
    q, s = per_token_quant_int8(xg.view(M, K))
    two = int8_scaled_mm(q, wg, s, sg.view(-1), dtype, bg)
    assert torch.equal(out.view(M, N).view(torch.int16), two.view(torch.int16))


def test_int8_linear_leaves_unusual_operands_to_the_operators(gpu):
    """Operands the one call does not take go through the two operators, which raise the reference's errors."""
    from sglang_amd.w8a8_int8 import apply_w8a8_int8_linear

    x = torch.randn(4, 512, device=gpu, dtype=torch.bfloat16)
    w_row_major = torch.zeros(512, 256, device=gpu, dtype=torch.int8)  # [K, N] but not column-major
    s = torch.ones(256, 1, device=gpu)
    with pytest.raises(RuntimeError, match="column major"):
        apply_w8a8_int8_linear(x, w_row_major, s)
    assert tuple(apply_w8a8_int8_linear(x[:0], w_row_major.t().contiguous().t(), s).shape) == (0, 256)
