"""GPU parity of every kernel variant behind the two GEMM entry points, with the route asserted.

Each shape of tests/gemm_cases.py is run through the public operator and compared with the CPU oracle in full; before
that the test asks the library which kernel it will use and checks that it is the variant the shape was chosen for
(tests/test_gemm_routes_cpu.py proves that the shapes between them reach every variant).  FP8 tolerance: see
tests/test_gpu_fp8_gemm.py; INT8: accumulators and outputs bit-exact.
"""
import pytest
import torch

from gemm_cases import FP8_ROUTE_SHAPES, INT8_ROUTE_SHAPES, plan_for, variant_of
from test_gpu_fp8_gemm import _check, _rand_fp8
from sglang_amd.workloads import cdiv

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


@pytest.mark.parametrize("M,N,K", FP8_ROUTE_SHAPES)
def test_fp8_variant_parity(gpu, oracle, M, N, K):
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul

    plan = plan_for("fp8", M, N, K)
    print(f"case fp8 M={M} N={N} K={K} -> {variant_of(plan, K)} {plan}", flush=True)
    g = torch.Generator().manual_seed(M * 131 + N * 7 + K)
    a, w = _rand_fp8((M, K), g), _rand_fp8((N, K), g)
    As = torch.rand(M, cdiv(K, 128), generator=g) * 1e-2 + 1e-4
    Bs = torch.rand(cdiv(N, 128), cdiv(K, 128), generator=g) * 1e-2 + 1e-4
    out = w8a8_block_fp8_matmul(a.to(gpu), w.to(gpu), As.to(gpu), Bs.to(gpu), [128, 128], torch.bfloat16)
    assert tuple(out.shape) == (M, N)
    rows = torch.arange(M) if M <= 512 else torch.cat(
        [torch.tensor([0, 1, 127, 128, 255, 256, 257, M - 257, M - 256, M - 2, M - 1]), torch.randperm(M, generator=g)[:40]])
    ref, mag = oracle.fp8_blockwise_mm(a[rows].contiguous(), w, As[rows].contiguous(), Bs, torch.float32, want_abs=True)
    _check(out[rows.to(gpu)], ref, mag, f"M={M} N={N} K={K}")
    assert bool(torch.isfinite(out).all())


EXACT_SHAPES = [s for s in FP8_ROUTE_SHAPES if s[1] % 128 == 0 and s[2] % 128 == 0]


@pytest.mark.parametrize("M,N,K", EXACT_SHAPES)
def test_fp8_variant_exact_integers(gpu, M, N, K):
    """Integer-valued codes and power-of-two scales: every product, block sum and promotion is exact in fp32 whatever
    the summation order, so each variant must reproduce integer arithmetic bit for bit - a stale LDS stage, a block
    multiplied twice or skipped, a wrong scale index or an early wait all show up as a wrong integer."""
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul

    print(f"case fp8-exact M={M} N={N} K={K} -> {variant_of(plan_for('fp8', M, N, K), K)}", flush=True)
    g = torch.Generator().manual_seed(M + 3 * N + 5 * K)
    ai = torch.randint(-8, 9, (M, K), generator=g)
    wi = torch.randint(-8, 9, (N, K), generator=g)
    sa = torch.exp2(torch.randint(-3, 4, (M, K // 128), generator=g).float())
    sw = torch.exp2(torch.randint(-3, 4, (N // 128, K // 128), generator=g).float())
    out = w8a8_block_fp8_matmul(ai.float().to(FP8).to(gpu), wi.float().to(FP8).to(gpu), sa.to(gpu), sw.to(gpu),
                                [128, 128], torch.float32)
    rows = torch.arange(M) if M <= 256 else torch.cat([torch.tensor([0, 255, 256, M - 1]), torch.randperm(M, generator=g)[:60]])
    # dequantize exactly (small integers times powers of two) and multiply in fp64: exact
    a_d = ai[rows].double() * sa[rows].double().repeat_interleave(128, dim=1)
    w_d = wi.double() * sw.double().repeat_interleave(128, dim=0).repeat_interleave(128, dim=1)
    want = a_d @ w_d.T
    assert torch.equal(out[rows.to(gpu)].cpu().double(), want), (M, N, K)


@pytest.mark.parametrize("M,N,K", INT8_ROUTE_SHAPES)
def test_int8_variant_parity(gpu, oracle, M, N, K):
    from sglang_amd import ops
    from sglang_amd.sgl_kernel import int8_scaled_mm

    plan = plan_for("int8", M, N, K)
    print(f"case int8 M={M} N={N} K={K} -> {variant_of(plan, K)} {plan}", flush=True)
    g = torch.Generator().manual_seed(M * 17 + N + K)
    a = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    sa, sb = torch.rand(M, generator=g) * 0.1, torch.rand(N, generator=g) * 0.01
    bias = (torch.randn(N, generator=g) * 10).to(torch.bfloat16)
    ag, wg = a.to(gpu), w.to(gpu)
    acc = ops.int8_mm_raw_accumulators(ag, wg.t())
    out = int8_scaled_mm(ag, wg.t(), sa.to(gpu), sb.to(gpu), torch.bfloat16, bias.to(gpu))
    rows = torch.arange(M) if M <= 512 else torch.cat(
        [torch.tensor([0, 31, 32, 127, 128, 255, 256, M - 257, M - 33, M - 2, M - 1]), torch.randperm(M, generator=g)[:24]])
    want_acc = oracle.int8_mm_acc(a[rows].contiguous(), w)
    assert torch.equal(acc[rows.to(gpu)].cpu(), want_acc)
    want = oracle.int8_epilogue(want_acc, sa[rows], sb, torch.bfloat16, bias)
    assert torch.equal(out[rows.to(gpu)].cpu().view(torch.int16), want.view(torch.int16))
