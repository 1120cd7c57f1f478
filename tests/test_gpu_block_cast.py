"""GPU parity of the weight-side 128 x 128 block (re)quantization: per_block_cast_to_fp8, block_quant_dequant,
quant_weight_ue8m0 and requant_weight_ue8m0 (python/sglang/srt/layers/quantization/fp8_utils.py:392-505) - codes, scales
and dequantized values bit-exact against the oracle, which is pinned on the CPU against the reference's own torch
formulation; the packed scale layout is checked byte by byte."""
import pytest
import torch

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def _bits(t):
    t = t.cpu()
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1024, 2048), (256, 384), (130, 200), (5, 7), (384, 1000), (129, 136)])
def test_block_cast_bits(gpu, oracle, dtype, shape):
    from sglang_amd.fp8_utils import per_block_cast_to_fp8

    g = torch.Generator().manual_seed(shape[0] + 3 * shape[1])
    x = (torch.randn(*shape, generator=g) * torch.rand(*shape, generator=g).pow(4) * 3).to(dtype)
    x[0, 0] = 448.0 * 0.25
    q, s = per_block_cast_to_fp8(x.to(gpu))
    q_o, s_o = oracle.block_cast_to_fp8(x)
    assert q.dtype == FP8 and tuple(s.shape) == tuple(s_o.shape)
    assert torch.equal(s.cpu(), s_o)
    assert torch.equal(_bits(q), q_o.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(512, 1024), (200, 300), (128, 136), (3, 5)])
def test_block_dequant_bits(gpu, oracle, dtype, shape):
    from sglang_amd.fp8_utils import block_quant_dequant

    n, k = shape
    g = torch.Generator().manual_seed(n + k)
    codes = torch.randint(0, 256, (n, k), generator=g, dtype=torch.uint8)
    codes = torch.where((codes & 0x7F) == 0x7F, codes & 0xF7, codes)
    s = torch.rand((n + 127) // 128, (k + 127) // 128, generator=g) * 0.01 + 1e-4
    out = block_quant_dequant(codes.view(FP8).to(gpu), s.to(gpu), [128, 128], dtype)
    ref = oracle.block_dequant_fp8(codes.view(FP8), s, dtype)
    assert out.dtype == dtype and torch.equal(_bits(out), _bits(ref))


def test_requant_weight_ue8m0(gpu, oracle):
    from sglang_amd.fp8_utils import requant_weight_ue8m0
    from sglang_amd.workloads import make_fp8_weight

    E, N, K = 2, 384, 640  # a stacked (expert) weight: leading batch dimension, K / 128 = 5 groups (one padded word)
    ws, ss = zip(*[make_fp8_weight(N, K, seed=40 + e) for e in range(E)])
    w, s = torch.stack(ws), torch.stack(ss)
    new_w, new_s = requant_weight_ue8m0(w.to(gpu), s.to(gpu), [128, 128])
    assert tuple(new_w.shape) == (E, N, K) and new_w.dtype == FP8
    assert tuple(new_s.shape) == (E, N, 2) and new_s.dtype == torch.int32 and new_s.stride(-2) == 1 and new_s.stride(-1) == N
    for e in range(E):
        deq = oracle.block_dequant_fp8(ws[e], ss[e], torch.bfloat16)
        q_o, s_o = oracle.block_cast_to_fp8(deq)
        assert torch.equal(_bits(new_w[e]), q_o.view(torch.uint8))
        words = torch.empty((N, 2), dtype=torch.int32)
        words.copy_(new_s[e].cpu())
        got = words.view(torch.uint8).reshape(N, 8)
        want = ((s_o.view(torch.int32) >> 23) & 0xFF).to(torch.uint8)  # [N/128, 5]
        assert torch.equal(got[:, :5], want.repeat_interleave(128, 0))
        assert not bool(got[:, 5:].any())
        # the requantized weight is close to the original one: power-of-two scales lose at most one bit of range
        orig = deq.float()
        back = oracle.block_dequant_fp8(q_o, s_o, torch.float32)
        assert float((back - orig).abs().max()) <= float(orig.abs().max()) * 2.0 ** -3
