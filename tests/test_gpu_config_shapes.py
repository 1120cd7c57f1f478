"""The benchmark configurations at their full sizes, against the CPU oracle.

Decode sizes (M <= 128) are compared in full; at M = 4096 the oracle checks a sample of rows (first, last, tile
borders, random) over all channels, which reaches every workgroup column and every K block.  Weights are drawn once
per (N, K) and shared by the cases that use them.  Tolerances as in tests/test_gpu_fp8_gemm.py (FP8) and bit-exact (INT8).
"""
import functools

import pytest
import torch

from gemm_cases import FP8_DECODE_CONFIG, FP8_PREFILL_CONFIG, INT8_CONFIG, plan_for, variant_of
from fp8_tolerance import FP8_MAG_TOL, FP8_MAG_TOL_CONFIG
from test_gpu_fp8_gemm import _check
from sglang_amd.workloads import cdiv, make_activation, make_fp8_weight

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def _codes(shape, g):
    c = torch.randint(0, 256, shape, generator=g, dtype=torch.uint8)
    return torch.where((c & 0x7F) == 0x7F, c & 0xF7, c).view(FP8)  # every finite e4m3fn code, no NaN


@functools.lru_cache(maxsize=2)
def _fp8_weight(N, K):
    g = torch.Generator().manual_seed(N * 10007 + K)
    return _codes((N, K), g), torch.rand(cdiv(N, 128), cdiv(K, 128), generator=g) * 1e-2 + 1e-4


@functools.lru_cache(maxsize=2)
def _int8_weight(N, K):
    g = torch.Generator().manual_seed(N * 10009 + K)
    return torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8), torch.rand(N, generator=g) * 0.01


def _sample_rows(M, g, tile=256):
    if M <= 512:
        return torch.arange(M)
    edge = torch.tensor([0, 1, tile - 1, tile, tile + 1, M // 2 - 1, M // 2, M - tile - 1, M - tile, M - 2, M - 1])
    return torch.cat([edge, torch.randperm(M, generator=g)[:37]])


@pytest.mark.parametrize("M,N,K", sorted(FP8_DECODE_CONFIG + FP8_PREFILL_CONFIG, key=lambda s: (s[1], s[2], s[0])))
def test_fp8_config_shape(gpu, oracle, M, N, K):
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul

    print(f"case fp8 M={M} N={N} K={K} -> {variant_of(plan_for('fp8', M, N, K), K)}", flush=True)
    w, Bs = _fp8_weight(N, K)
    g = torch.Generator().manual_seed(M)
    a = _codes((M, K), g)
    As = torch.rand(M, cdiv(K, 128), generator=g) * 1e-2 + 1e-4
    out = w8a8_block_fp8_matmul(a.to(gpu), w.to(gpu), As.to(gpu), Bs.to(gpu), [128, 128], torch.bfloat16)
    rows = _sample_rows(M, g)
    ref, mag = oracle.fp8_blockwise_mm(a[rows].contiguous(), w, As[rows].contiguous(), Bs, torch.float32, want_abs=True)
    _check(out[rows.to(gpu)], ref, mag, f"M={M} N={N} K={K}")
    assert bool(torch.isfinite(out).all())


@functools.lru_cache(maxsize=1)
def _config_weight(N, K):
    return make_fp8_weight(N, K)


@pytest.mark.parametrize("M,N,K", sorted(FP8_DECODE_CONFIG + FP8_PREFILL_CONFIG, key=lambda s: (s[1], s[2], s[0])))
def test_fp8_config_shape_on_its_own_distribution(gpu, oracle, M, N, K):
    """The same shapes on the operands the configurations describe: N(0,1) activations with 0.1 % outliers x 50 through
    the GPU quantizer (1 x 128 groups; codes and scales equal the oracle's bit for bit, asserted on the sampled rows),
    N(0, 0.02) weights quantized per 128 x 128 block.  Scale magnitudes and cancellation differ from uniformly random
    codes, so the tolerance constant is the one measured for this distribution (tests/fp8_tolerance.py)."""
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8
    from sglang_amd.fp8_utils import dispatch_w8a8_block_fp8_linear

    print(f"case fp8 M={M} N={N} K={K} -> {variant_of(plan_for('fp8', M, N, K), K)}", flush=True)
    w_q, w_s = _config_weight(N, K)
    x = make_activation(M, K)
    # the linear method's forward: `x / s` codes with M-major scales, or, for N = 576 (not a multiple of 128), the
    # fallback with `x * (1 / s)` codes and row-major scales
    aligned = N % 128 == 0
    out = dispatch_w8a8_block_fp8_linear()(x.to(gpu), w_q.to(gpu), [128, 128], w_s.to(gpu))
    x_q, x_s = per_token_group_quant_fp8(x.to(gpu), 128, column_major_scales=aligned)
    g = torch.Generator().manual_seed(M)
    rows = _sample_rows(M, g)
    q_o, s_o = oracle.group_quant(x[rows].contiguous(), 128, mode="div" if aligned else "rcp")
    assert torch.equal(x_q[rows.to(gpu)].cpu().view(torch.uint8), q_o.view(torch.uint8))
    assert torch.equal(x_s[rows.to(gpu)].cpu(), s_o)
    ref, mag = oracle.fp8_blockwise_mm(q_o, w_q, s_o, w_s, torch.float32, want_abs=True)
    _check(out[rows.to(gpu)], ref, mag, f"config distribution M={M} N={N} K={K}",
           mag_tol=FP8_MAG_TOL_CONFIG if K >= 1536 else FP8_MAG_TOL, min_pure=0.997)
    assert bool(torch.isfinite(out).all())


@pytest.mark.parametrize("M,N,K", sorted(INT8_CONFIG, key=lambda s: (s[1], s[2], s[0])))
def test_int8_config_shape(gpu, oracle, M, N, K):
    from sglang_amd import ops
    from sglang_amd.sgl_kernel import int8_scaled_mm

    print(f"case int8 M={M} N={N} K={K} -> {variant_of(plan_for('int8', M, N, K), K)}", flush=True)
    w, sb = _int8_weight(N, K)
    g = torch.Generator().manual_seed(M)
    a = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8)
    sa = torch.rand(M, generator=g) * 0.1
    bias = (torch.randn(N, generator=g) * 10).to(torch.bfloat16)
    ag, wg = a.to(gpu), w.to(gpu)
    acc = ops.int8_mm_raw_accumulators(ag, wg.t())
    out = int8_scaled_mm(ag, wg.t(), sa.to(gpu), sb.to(gpu), torch.bfloat16, bias.to(gpu))
    rows = _sample_rows(M, g)
    want_acc = oracle.int8_mm_acc(a[rows].contiguous(), w)
    assert torch.equal(acc[rows.to(gpu)].cpu(), want_acc)
    want = oracle.int8_epilogue(want_acc, sa[rows], sb, torch.bfloat16, bias)
    assert torch.equal(out[rows.to(gpu)].cpu().view(torch.int16), want.view(torch.int16))
