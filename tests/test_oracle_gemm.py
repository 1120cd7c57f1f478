"""Pins the oracle's GEMMs against torch CPU matmuls and exact integer arithmetic.

  * blockwise FP8: the broadcast-scales fp64 matmul of the reference's kernel test
    (sgl-kernel/tests/test_fp8_blockwise_gemm.py:19-59), the tile loop of its Python test
    (python/sglang/test/test_block_fp8.py:273-325), and special cases whose answer is an
    exact integer (unit scales, integer-valued codes) so that a transposed operand, a
    dropped K block or a wrong scale index cannot pass;
  * INT8: int64 matmul (exact) and the three fp32 epilogue orders written with torch ops.
"""
import pytest
import torch

from sglang_amd.workloads import block_cast_to_fp8, cdiv, make_int8_activation, make_int8_weight

FP8 = torch.float8_e4m3fn


def _rand_fp8(shape, g):
    x = (torch.rand(*shape, generator=g) - 0.5) * 2 * 448.0
    return x.clamp(-448, 448).to(FP8)


def _broadcast_scaled_mm_f64(a, w, sa, sw):
    """(a * sa broadcast over 128 columns) @ (w * sw broadcast over 128x128 blocks).T in fp64."""
    M, K = a.shape
    N = w.shape[0]
    sa_full = sa.to(torch.float64).repeat_interleave(128, dim=1)[:, :K]
    sw_full = sw.to(torch.float64).repeat_interleave(128, dim=0)[:N].repeat_interleave(128, dim=1)[:, :K]
    return (a.to(torch.float64) * sa_full) @ (w.to(torch.float64) * sw_full).T


def _tile_loop_f32(a, w, sa, sw):
    M, K = a.shape
    N = w.shape[0]
    A, B = a.to(torch.float32), w.to(torch.float32)
    C = torch.zeros(M, N)
    for i in range(cdiv(K, 128)):
        for j in range(cdiv(N, 128)):
            ks, ns = slice(i * 128, min((i + 1) * 128, K)), slice(j * 128, min((j + 1) * 128, N))
            C[:, ns] += (A[:, ks] @ B[ns, ks].T) * (sa[:, i : i + 1] * sw[j, i])
    return C


@pytest.mark.parametrize("M,N,K", [(1, 128, 128), (5, 256, 512), (16, 1088, 512), (33, 200, 300), (7, 576, 1024)])
def test_fp8_blockwise_vs_torch(oracle, M, N, K):
    g = torch.Generator().manual_seed(M * 1000 + N + K)
    a, w = _rand_fp8((M, K), g), _rand_fp8((N, K), g)
    sa = torch.rand(M, cdiv(K, 128), generator=g) * 1e-2 + 1e-4
    sw = torch.rand(cdiv(N, 128), cdiv(K, 128), generator=g) * 1e-2 + 1e-4
    out, mag = oracle.fp8_blockwise_mm(a, w, sa, sw, torch.float32, want_abs=True)
    ref64 = _broadcast_scaled_mm_f64(a, w, sa, sw)
    # fp32 promotion of ~K/128 block sums: error is a few ulp of the magnitude sum
    assert bool(((out.to(torch.float64) - ref64).abs() <= 4e-7 * mag.to(torch.float64)).all())
    torch.testing.assert_close(out, _tile_loop_f32(a, w, sa, sw), rtol=2e-5, atol=1e-5 * float(mag.max()))
    # bf16 / fp16 outputs are the RNE casts of the fp32 result
    assert torch.equal(oracle.fp8_blockwise_mm(a, w, sa, sw, torch.bfloat16), out.to(torch.bfloat16))
    assert torch.equal(oracle.fp8_blockwise_mm(a, w, sa * 1e-3, sw, torch.float16),
                       oracle.fp8_blockwise_mm(a, w, sa * 1e-3, sw, torch.float32).to(torch.float16))


def test_fp8_blockwise_exact_integer_case(oracle):
    # integer-valued codes in [-8, 8] and power-of-two scales: every product, block sum and
    # promotion is exact, so the result must equal integer arithmetic bit for bit.
    g = torch.Generator().manual_seed(4)
    M, N, K = 9, 384, 640
    ai = torch.randint(-8, 9, (M, K), generator=g)
    wi = torch.randint(-8, 9, (N, K), generator=g)
    sa_e = torch.randint(-3, 4, (M, K // 128), generator=g)
    sw_e = torch.randint(-3, 4, (N // 128, K // 128), generator=g)
    sa, sw = torch.exp2(sa_e.float()), torch.exp2(sw_e.float())
    out = oracle.fp8_blockwise_mm(ai.float().to(FP8), wi.float().to(FP8), sa, sw, torch.float32)
    want = torch.zeros(M, N, dtype=torch.float64)
    for kb in range(K // 128):
        part = (ai[:, kb * 128 : (kb + 1) * 128] @ wi[:, kb * 128 : (kb + 1) * 128].T).to(torch.float64)
        want += part * sa[:, kb : kb + 1].double() * sw[:, kb].double().repeat_interleave(128)[None, :]
    assert torch.equal(out.to(torch.float64), want)


def test_fp8_blockwise_strided_scales_and_operands(oracle):
    # the sgl_kernel entry takes M-major scales_a and K-major scales_b (transposed views); results must not depend on strides
    g = torch.Generator().manual_seed(8)
    M, N, K = 6, 256, 384
    a, w = _rand_fp8((M, K), g), _rand_fp8((N, K), g)
    sa = torch.rand(M, 3, generator=g)
    sw = torch.rand(2, 3, generator=g)
    base = oracle.fp8_blockwise_mm(a, w, sa, sw, torch.float32)
    sa_t = sa.t().contiguous().t()
    sw_t = sw.t().contiguous().t()
    assert sa_t.stride() == (1, M) and sw_t.stride() == (1, 2)
    assert torch.equal(oracle.fp8_blockwise_mm(a, w, sa_t, sw_t, torch.float32), base)
    a_pad = torch.zeros(M, K + 64, dtype=torch.uint8).view(FP8)
    a_pad[:, :K] = a
    assert torch.equal(oracle.fp8_blockwise_mm(a_pad[:, :K], w, sa, sw, torch.float32), base)


def test_fp8_blockwise_with_real_quantized_operands(oracle):
    # end to end: quantize a bf16 linear, run the blockwise GEMM, compare with the fp32 linear
    g = torch.Generator().manual_seed(12)
    M, N, K = 16, 256, 1024
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g) * 0.02
    wq, ws = block_cast_to_fp8(w)
    xq, xs = oracle.group_quant(x, 128, mode="div")
    out = oracle.fp8_blockwise_mm(xq, wq, xs, ws, torch.float32)
    ref = x.float() @ w.T
    rel = (out - ref).norm() / ref.norm()
    assert float(rel) < 0.06  # two fp8 roundings, ~2^-4 relative each, averaged over K


@pytest.mark.parametrize("M,N,K", [(1, 16, 512), (17, 200, 64), (64, 96, 1024)])
def test_int8_acc_exact(oracle, M, N, K):
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    acc = oracle.int8_mm_acc(a, w)
    assert torch.equal(acc.to(torch.int64), a.to(torch.int64) @ w.to(torch.int64).T)


def test_int8_acc_extremes(oracle):
    K = 14336
    a = torch.full((2, K), -128, dtype=torch.int8)
    w = torch.full((3, K), -128, dtype=torch.int8)
    w[1] = 127
    acc = oracle.int8_mm_acc(a, w)
    assert acc[0].tolist() == [128 * 128 * K, -128 * 127 * K, 128 * 128 * K]


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("with_bias", [False, True])
def test_int8_epilogue_orders(oracle, out_dtype, with_bias):
    g = torch.Generator().manual_seed(77)
    M, N, K = 24, 136, 512
    a, sa = make_int8_activation(M, K, seed=1)
    w, sb = make_int8_weight(N, K, seed=2)
    bias = (torch.randn(N, generator=g) * 10).to(out_dtype) if with_bias else None
    acc = oracle.int8_mm_acc(a, w)
    f = acc.to(torch.float32)
    sav, sbv = sa.view(-1, 1), sb.view(1, -1)
    b = bias.to(torch.float32) if with_bias else 0.0
    want = {
        oracle.EPI_COL_ROW: f * (sbv * sav) + b,
        oracle.EPI_ROW_COL_ACC: sav * (sbv * f) + b,
        oracle.EPI_TORCH: (f * sav) * sbv + b,
    }
    outs = {}
    for order, ref in want.items():
        outs[order] = oracle.int8_epilogue(acc, sa, sb, out_dtype, bias, order)
        assert torch.equal(outs[order], ref.to(out_dtype)), order
    # the orders differ only by fp32 rounding: at most one unit in the last place after the cast
    base = outs[oracle.EPI_COL_ROW].view(torch.int16).to(torch.int32)
    for order in (oracle.EPI_ROW_COL_ACC, oracle.EPI_TORCH):
        assert int((outs[order].view(torch.int16).to(torch.int32) - base).abs().max()) <= 1
    assert torch.equal(oracle.int8_scaled_mm(a, w, sa, sb, out_dtype, bias), outs[oracle.EPI_COL_ROW])


# ---------------------------------------------------------------- per-token x per-channel FP8 GEMM

def test_fp8_scaled_mm_against_fp64_matmul(oracle):
    """sgl-kernel/tests/test_fp8_gemm.py:7-15 in fp64: the oracle's exact sum, scaled as sa * (sb * acc) in fp32, may
    differ from fp64 by fp32 rounding only."""
    g = torch.Generator().manual_seed(11)
    M, N, K = 13, 40, 1000
    a = ((torch.rand(M, K, generator=g) - 0.5) * 896).to(torch.float8_e4m3fn)
    w = ((torch.rand(N, K, generator=g) - 0.5) * 896).to(torch.float8_e4m3fn)
    sa, sb = torch.randn(M, generator=g) * 1e-3, torch.randn(N, generator=g) * 1e-3
    bias = torch.randn(N, generator=g)
    out = oracle.fp8_scaled_mm(a, w, sa, sb, torch.float32, bias)
    ref = (a.double() @ w.double().T) * sa.double()[:, None] * sb.double()[None, :] + bias.double()[None, :]
    assert float(((out.double() - ref).abs() / (ref.abs() + 1e-30)).max()) < 1e-5
    # and the magnitude matrix bounds the result
    out2, mag = oracle.fp8_scaled_mm(a, w, sa, sb, torch.float32, None, want_abs=True)
    assert bool((out2.abs() <= mag * (1 + 1e-5)).all())


def test_fp8_scaled_mm_exact_integers_and_cast(oracle):
    g = torch.Generator().manual_seed(12)
    M, N, K = 9, 24, 384
    ai, wi = torch.randint(-8, 9, (M, K), generator=g), torch.randint(-8, 9, (N, K), generator=g)
    sa = torch.exp2(torch.randint(-3, 4, (M,), generator=g).float())
    sb = torch.exp2(torch.randint(-3, 4, (N,), generator=g).float())
    bias = torch.randint(-16, 17, (N,), generator=g).float().to(torch.bfloat16)
    out = oracle.fp8_scaled_mm(ai.float().to(torch.float8_e4m3fn), wi.float().to(torch.float8_e4m3fn), sa, sb, torch.bfloat16, bias)
    want = ((ai @ wi.T).double() * sa.double()[:, None] * sb.double()[None, :] + bias.double()[None, :]).to(torch.bfloat16)
    assert torch.equal(out, want)
