"""GPU parity of the blockwise FP8 GEMM with packed power-of-two (UE8M0) scales on both operands
(mi355_fp8_blockwise_mm_ue8m0; the reference's w8a8_block_fp8_matmul_deepgemm / deepgemm_w8a8_block_fp8_linear_with_fallback,
python/sglang/srt/layers/quantization/fp8_kernel.py:1047-1065, fp8_utils.py:217-255).

The oracle is the blockwise GEMM oracle fed with the decoded scales 2^(byte - 127).  Floating point:
|out - ref| <= 1e-2 * |ref| + 1e-4 * mag, as for the fp32-scale GEMM (tests/test_gpu_fp8_gemm.py); with small-integer
operands every product and partial sum is exact in fp32 and the result must match bit for bit, whichever kernel runs.
Large shapes, mid-M shapes (every tile and split of the three-stage kernel) and decode shapes on the wave-split kernel
take kernels whose MFMA applies the scales itself, the others the fp32-scale kernels behind an unpack step; all are covered, and so are K extents whose last exponent word is only partly used."""
import pytest
import torch

from fp8_tolerance import check_fp8_gemm
from sglang_amd.workloads import make_activation, make_fp8_weight

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn

# (M, N, K): two-phase kernel with hardware scales (>= 256 tiles of 256 x 256): K of 4, 9 and 5 blocks; ragged M;
# then decode, mid-M, generic routes through the unpack step
# decode sizes on the wave-split kernel, which also lets the MFMA apply the scales (8 and 4 waves, a ragged last round and a
# partly used last exponent word: K = 4480 is 35 blocks; N = 576 is not a multiple of 128), then the same kernel with two
# channel tiles per workgroup (8 waves with one round and two, 4 waves with one round and many)
SHAPES = [(4096, 4352, 512), (4096, 4352, 1152), (4000, 4352, 640), (4, 512, 1024), (16, 2048, 7168), (200, 16384, 2048),
          (50, 384, 512), (1500, 640, 1024), (2, 2048, 7168), (3, 1536, 4480), (1, 1024, 18432), (5, 576, 2048),
          (7, 6432, 4096), (12, 18432, 7168), (6, 16640, 4480), (5, 36864, 1280), (1, 7168, 18432), (16, 7168, 36864),
          (3990, 4224, 640)]  # two-phase kernel: a last token tile with 6 of 16 rows and half a last channel tile (guarded stores)


def _unpack_bytes(words, groups):
    dense = torch.empty(tuple(words.shape), dtype=torch.int32)
    dense.copy_(words.cpu())
    return dense.view(torch.uint8).reshape(words.shape[0], -1)[:, :groups]


def _operands(M, N, K, gpu, seed):
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.fp8_utils import requant_weight_ue8m0

    w_q, w_s = make_fp8_weight(N, K, seed=seed)
    w2, sb_words = requant_weight_ue8m0(w_q.to(gpu), w_s.to(gpu), [128, 128])
    x = make_activation(M, K, seed=seed + 1).to(gpu)
    x_q, sa_words = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True,
                                                     enable_v2=True)
    return x_q, sa_words, w2, sb_words


def _reference(oracle, x_q, sa_words, w2, sb_words, rows=None):
    K = x_q.shape[1]
    KB = K // 128
    sa = torch.exp2(_unpack_bytes(sa_words, KB).float() - 127.0)
    sb = torch.exp2(_unpack_bytes(sb_words, KB).float() - 127.0)[::128].contiguous()
    a = x_q.cpu()
    if rows is not None:
        a, sa = a[rows].contiguous(), sa[rows].contiguous()
    return oracle.fp8_blockwise_mm(a, w2.cpu(), sa.contiguous(), sb, torch.float32, want_abs=True)


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_ue8m0_gemm_against_oracle(gpu, oracle, M, N, K):
    from sglang_amd import _lib
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul_deepgemm

    print(f"case M={M} N={N} K={K} -> {_lib.gemm_plan('fp8', M, N, K)['kernel']}", flush=True)
    x_q, sa_words, w2, sb_words = _operands(M, N, K, gpu, 3 * M + N + K)
    out = w8a8_block_fp8_matmul_deepgemm(x_q, w2, sa_words, sb_words, [128, 128], torch.bfloat16)
    assert tuple(out.shape) == (M, N) and out.dtype == torch.bfloat16
    g = torch.Generator().manual_seed(M)
    rows = torch.arange(M) if M <= 256 else torch.cat([torch.tensor([0, 127, 128, 255, 256, M - 1]), torch.randperm(M, generator=g)[:26]])
    ref, mag = _reference(oracle, x_q, sa_words, w2, sb_words, rows)
    check_fp8_gemm(out[rows.to(gpu)], ref, mag, f"M={M} N={N} K={K}")


@pytest.mark.parametrize("M,N,K", [(4096, 4352, 1152), (16, 2048, 1024), (200, 16384, 640), (2, 2048, 1152), (3, 144, 4480)])
def test_ue8m0_gemm_exact_integers(gpu, oracle, M, N, K):
    """Operands in {-2..2}, exponents in a narrow band: every block product and every partial sum is an integer times a
    power of two well inside fp32, so any summation order gives the same bits."""
    from sglang_amd import ops

    g = torch.Generator().manual_seed(K + M)
    a = torch.randint(-2, 3, (M, K), generator=g).float().to(FP8)
    w = torch.randint(-2, 3, (N, K), generator=g).float().to(FP8)
    KB, KW = K // 128, (K // 128 + 3) // 4
    ea = torch.randint(120, 129, (M, KB), generator=g, dtype=torch.uint8)
    eb = torch.randint(122, 131, ((N + 127) // 128, KB), generator=g, dtype=torch.uint8)

    def pack(e, rows_out, repeat):  # [R, KB] bytes -> int32 [rows_out, KW] with stride(0) == 1
        full = torch.zeros(e.shape[0], KW * 4, dtype=torch.uint8)
        full[:, :KB] = e
        words = full.view(torch.int32).repeat_interleave(repeat, 0)[:rows_out]           # [rows, KW]
        pad = (rows_out + 3) // 4 * 4
        buf = torch.zeros(KW, pad, dtype=torch.int32)
        buf[:, :rows_out] = words.t()
        return buf

    sa_buf, sb_buf = pack(ea, M, 1).to(gpu), pack(eb, N, 128).to(gpu)
    sa_words, sb_words = sa_buf.t()[:M], sb_buf.t()[:N]
    out = ops.fp8_blockwise_mm_ue8m0(a.to(gpu), w.to(gpu), sa_words, sb_words, torch.bfloat16)
    ref = oracle.fp8_blockwise_mm(a, w, torch.exp2(ea.float() - 127), torch.exp2(eb.float() - 127), torch.bfloat16)
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


# one shape per tile (64 / 128 tokens x 128 / 192 / 256 channels) and split of the mid-M kernel, which applies the exponents
# in the MFMA too; 50 x 3000 has a ragged last channel tile, 33 x 16384 x 2176 a last exponent word with one byte used
MID_M = [(48, 16384, 2048), (33, 16384, 2176), (40, 4096, 7168), (50, 3000, 4224), (24, 36864, 14336), (130, 3072, 7168), (40, 65536, 512),
         (130, 4096, 7168), (100, 32768, 640), (65, 7168, 18432), (100, 36864, 640), (300, 3072, 14336), (100, 65536, 512),
         (400, 4096, 16384),
         (14, 36864, 1280), (16, 65536, 1152), (8, 36864, 7168), (16, 24576, 1536)]  # decode sizes on one round of unsplit 64-token tiles


def test_mid_m_shapes_reach_every_tile_and_split():
    from sglang_amd import _lib

    reached = set()
    for M, N, K in MID_M:
        p = _lib.gemm_plan("fp8", M, N, K)
        assert p["kernel"] == "dma3", (M, N, K, p)
        reached.add((p["bm"], p["bn"], p["splits"] > 1))
    assert reached == {(bm, bn, sp) for bm in (64, 128) for bn in (128, 192, 256) for sp in (False, True)}


@pytest.mark.parametrize("M,N,K", MID_M)
def test_ue8m0_mid_m_kernel_against_oracle(gpu, oracle, M, N, K):
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul_deepgemm

    x_q, sa_words, w2, sb_words = _operands(M, N, K, gpu, M + 7 * N + K)
    out = w8a8_block_fp8_matmul_deepgemm(x_q, w2, sa_words, sb_words, [128, 128], torch.bfloat16)
    rows = torch.arange(M) if M <= 64 else torch.cat([torch.tensor([0, 63, 64, min(127, M - 1), M - 1]),
                                                       torch.randperm(M, generator=torch.Generator().manual_seed(M))[:27]])
    ref, mag = _reference(oracle, x_q, sa_words, w2, sb_words, rows)
    check_fp8_gemm(out[rows.to(gpu)], ref, mag, f"M={M} N={N} K={K}")


# the streaming decode kernel: one K range and several, the last range short (K blocks not a multiple of 8), one to four
# bytes used in the last exponent word, token counts below and at the 16 rows of the MFMA tile (rows past M repeat the last token)
DECODE = [(8, 256, 512), (4, 4352, 512), (5, 4096, 36864), (16, 4096, 36864), (13, 18432, 7168), (15, 18432, 7168), (9, 3072, 1536),
          (14, 70656, 1280), (14, 16384, 2304), (15, 65536, 640), (16, 66560, 1152), (13, 4096, 18432), (8, 4352, 128)]


def test_decode_shapes_reach_the_streaming_kernel():
    from sglang_amd import _lib

    plans = [_lib.gemm_plan("fp8", M, N, K) for M, N, K in DECODE]
    assert all(p["kernel"] == "decode" for p in plans), plans
    assert {p["splits"] > 1 for p in plans} == {False, True}


@pytest.mark.parametrize("M,N,K", DECODE)
def test_ue8m0_decode_kernel_against_oracle(gpu, oracle, M, N, K):
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul_deepgemm

    x_q, sa_words, w2, sb_words = _operands(M, N, K, gpu, 3 * M + N + 5 * K)
    out = w8a8_block_fp8_matmul_deepgemm(x_q, w2, sa_words, sb_words, [128, 128], torch.bfloat16)
    ref, mag = _reference(oracle, x_q, sa_words, w2, sb_words)
    check_fp8_gemm(out, ref, mag, f"M={M} N={N} K={K}")


def _exact_integer_case(gpu, oracle, M, N, K):
    """Small-integer operands and exponents drawn anew for every token, weight block and K block from a narrow band: exact in
    fp32, so the MFMA-applied scales (each byte of each word in its place), the fp32 partial sums and their ordered reduce
    must reproduce the oracle's bits."""
    from sglang_amd import ops

    g = torch.Generator().manual_seed(K + M)
    a = torch.randint(-2, 3, (M, K), generator=g).float().to(FP8)
    w = torch.randint(-2, 3, (N, K), generator=g).float().to(FP8)
    KB, KW = K // 128, (K // 128 + 3) // 4
    ea = torch.randint(124, 129, (M, KB), generator=g, dtype=torch.uint8)
    eb = torch.randint(124, 129, ((N + 127) // 128, KB), generator=g, dtype=torch.uint8)

    def pack(e, rows_out, repeat):
        full = torch.zeros(e.shape[0], KW * 4, dtype=torch.uint8)
        full[:, :KB] = e
        words = full.view(torch.int32).repeat_interleave(repeat, 0)[:rows_out]
        buf = torch.zeros(KW, (rows_out + 3) // 4 * 4, dtype=torch.int32)
        buf[:, :rows_out] = words.t()
        return buf

    sa_buf, sb_buf = pack(ea, M, 1).to(gpu), pack(eb, N, 128).to(gpu)
    out = ops.fp8_blockwise_mm_ue8m0(a.to(gpu), w.to(gpu), sa_buf.t()[:M], sb_buf.t()[:N], torch.bfloat16)
    ref = oracle.fp8_blockwise_mm(a, w, torch.exp2(ea.float() - 127), torch.exp2(eb.float() - 127), torch.bfloat16)
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("M,N,K", [(130, 3072, 7168), (65, 7168, 18432), (100, 36864, 640)])
def test_ue8m0_mid_m_exact_integers(gpu, oracle, M, N, K):
    _exact_integer_case(gpu, oracle, M, N, K)  # split and unsplit mid-M plans


@pytest.mark.parametrize("M,N,K", [(8, 4352, 512), (13, 18432, 7168), (16, 2048, 7168), (14, 16384, 2304), (5, 4096, 36864)])
def test_ue8m0_decode_exact_integers(gpu, oracle, M, N, K):
    from sglang_amd import _lib

    assert _lib.gemm_plan("fp8", M, N, K)["kernel"] == "decode"
    _exact_integer_case(gpu, oracle, M, N, K)


@pytest.mark.parametrize("M,N,K", [(8, 4352, 512), (4096, 4352, 512), (12, 2048, 7168), (200, 1024, 640), (8, 36864, 1152)])
def test_deepgemm_linear_wrapper(gpu, oracle, M, N, K):
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8, w8a8_block_fp8_matmul_deepgemm
    from sglang_amd.fp8_utils import deepgemm_w8a8_block_fp8_linear_with_fallback, requant_weight_ue8m0

    w_q, w_s = make_fp8_weight(N, K, seed=9)
    w2, sb_words = requant_weight_ue8m0(w_q.to(gpu), w_s.to(gpu), [128, 128])
    x = make_activation(M, K, seed=10)
    bias = torch.randn(N, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    out = deepgemm_w8a8_block_fp8_linear_with_fallback(x.to(gpu).view(M // 4, 4, K), w2, [128, 128], sb_words, None, bias.to(gpu))
    assert tuple(out.shape) == (M // 4, 4, N) and out.dtype == torch.bfloat16
    v = x.clone()
    q_o, s_o = oracle.group_quant(v, 128, mode="mul", layout="ue8m0")
    sa = torch.exp2(oracle.unpack_ue8m0(s_o, K // 128).float() - 127.0)
    sb = torch.exp2(_unpack_bytes(sb_words, K // 128).float() - 127.0)[::128].contiguous()
    rows = torch.arange(M) if M <= 64 else torch.tensor([0, 1, 255 % M, 256 % M, M - 1])
    ref, mag = oracle.fp8_blockwise_mm(q_o[rows].contiguous(), w2.cpu(), sa[rows].contiguous(), sb, torch.float32, want_abs=True)
    # the wrapper rounds the product to bf16 and then adds the bias (fp8_utils.py:250-254): up to half a unit in the last place of the product, 2^-8 of it
    check_fp8_gemm(out.reshape(M, N)[rows.to(gpu)], ref + bias.float()[None, :], mag, "deepgemm linear", extra=2.0 ** -8 * ref.abs())
    # the wrapper's one C-ABI call against its two calls through the operator entry points: the same bits
    plain = deepgemm_w8a8_block_fp8_linear_with_fallback(x.to(gpu), w2, [128, 128], sb_words)
    q, s = sglang_per_token_group_quant_fp8(x.to(gpu), 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True,
                                            enable_v2=True)
    two = w8a8_block_fp8_matmul_deepgemm(q, w2, s, sb_words, [128, 128], torch.bfloat16)
    assert torch.equal(plain.view(torch.int16), two.view(torch.int16))
    # an fp32 block scale tensor (a checkpoint that was not re-quantized) takes the ordinary block-FP8 linear
    out2 = deepgemm_w8a8_block_fp8_linear_with_fallback(x.to(gpu), w_q.to(gpu), [128, 128], w_s.to(gpu), None, None)
    assert tuple(out2.shape) == (M, N)


@pytest.mark.parametrize("M,N,K", [(4096, 4352, 512), (16, 2048, 1024), (6, 640, 1152), (200, 1024, 640)])
def test_w8a8_block_fp8_matmul_takes_packed_scales(gpu, oracle, M, N, K):
    """python/sglang/srt/layers/quantization/fp8_kernel.py:1016-1019, :1034-1039: `w8a8_block_fp8_matmul` and
    `prepare_block_fp8_matmul_inputs` accept scales packed as UE8M0 exponent bytes in int32 words, [..., ceil(K/512)] for
    the activation and [N, ceil(K/512)] for the weight.  With both operands packed the result is the UE8M0 kernel's, bit
    for bit, for 2-D and batched activations and for token words that are not packed along tokens; with one side packed
    and the other fp32 the packed side is expanded first and the result is held against the oracle."""
    from sglang_amd.fp8_kernel import prepare_block_fp8_matmul_inputs, w8a8_block_fp8_matmul, w8a8_block_fp8_matmul_deepgemm

    x_q, sa_words, w2, sb_words = _operands(M, N, K, gpu, 5 * M + N + K)
    assert sa_words.dtype == torch.int32 and tuple(sa_words.shape) == (M, (K // 128 + 3) // 4)
    assert prepare_block_fp8_matmul_inputs(x_q, w2, sa_words, sb_words, [128, 128], torch.bfloat16)[:3] == (M, N, K)
    want = w8a8_block_fp8_matmul_deepgemm(x_q, w2, sa_words, sb_words, [128, 128], torch.bfloat16)
    got = w8a8_block_fp8_matmul(x_q, w2, sa_words, sb_words, [128, 128], torch.bfloat16)
    assert got.dtype == torch.bfloat16 and torch.equal(got.view(torch.int16), want.view(torch.int16))
    # words stored row-major instead of along tokens, and a leading batch dimension
    got = w8a8_block_fp8_matmul(x_q.view(2, M // 2, K), w2, sa_words.contiguous().view(2, M // 2, -1), sb_words, [128, 128], torch.bfloat16)
    assert tuple(got.shape) == (2, M // 2, N) and torch.equal(got.view(M, N).view(torch.int16), want.view(torch.int16))
    g = torch.Generator().manual_seed(M)
    rows = torch.arange(M) if M <= 256 else torch.cat([torch.tensor([0, 255, 256, M - 1]), torch.randperm(M, generator=g)[:28]])
    ref, mag = _reference(oracle, x_q, sa_words, w2, sb_words, rows)
    KB = K // 128
    sa_f32 = torch.exp2(_unpack_bytes(sa_words, KB).float() - 127.0).to(gpu)
    sb_f32 = torch.exp2(_unpack_bytes(sb_words, KB).float() - 127.0)[::128].contiguous().to(gpu)
    for As, Bs in ((sa_words, sb_f32), (sa_f32, sb_words)):
        mixed = w8a8_block_fp8_matmul(x_q, w2, As, Bs, [128, 128], torch.float16)
        assert mixed.dtype == torch.float16
        check_fp8_gemm(mixed[rows.to(gpu)], ref, mag, f"mixed scales M={M} N={N} K={K}")
    with pytest.raises(AssertionError):
        w8a8_block_fp8_matmul(x_q, w2, sa_words[:, :0], sb_words, [128, 128], torch.bfloat16)
