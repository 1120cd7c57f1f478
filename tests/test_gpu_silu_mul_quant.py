"""GPU parity of silu(gate) * up fused in front of the group quantizer (sgl_per_token_group_quant_8bit_v2 with
fuse_silu_and_mul, plain and masked layouts): codes and packed UE8M0 scale bytes bit-exact against the oracle
(oracle.silu_mul, then oracle.group_quant in the v2 arithmetic).  Bit-exact is possible because the kernel and the oracle
evaluate exp by the same sequence of fp32 operations; against the reference's definition (approximate GPU exp) the
oracle itself is pinned on the CPU with the reference's kind of tolerance (tests/test_oracle_quant.py).

Shapes follow sgl-kernel/tests/test_per_token_group_quant_8bit.py:62-99 (hidden 2048, group 128, masked layouts
balanced / imbalanced / extreme), scaled down in the number of experts and padded tokens so that the CPU side stays fast.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def _data(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(*shape, generator=g)
    x[torch.randn(*shape, generator=g) < -2.5] *= 10  # outliers, as the reference's test data has
    return x.to(dtype)


def _expect(oracle, x2d):
    """[rows, 2H] -> codes [rows, H] uint8, exponent bytes [rows, H/128] uint8."""
    v = oracle.silu_mul(x2d)
    q, s = oracle.group_quant(v, 128, mode="mul", layout="ue8m0")
    return q.view(torch.uint8), oracle.unpack_ue8m0(s, v.shape[1] // 128)


def _scale_bytes(x_s, G):
    """packed int32 [T, words] with any strides -> uint8 [T, G]"""
    dense = torch.empty(tuple(x_s.shape), dtype=torch.int32)
    dense.copy_(x_s.cpu())
    return dense.view(torch.uint8).reshape(x_s.shape[0], -1)[:, :G]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H", [(1, 128), (4, 2048), (33, 2048), (512, 2048), (7, 640), (64, 7168), (5, 3200)])
def test_fused_plain_layout(gpu, oracle, dtype, T, H):
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8

    x = _data((T, 2 * H), dtype, 31 * T + H)
    x_q, x_s = sglang_per_token_group_quant_fp8(
        x.to(gpu), 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True, fuse_silu_and_mul=True,
        enable_v2=True)
    assert tuple(x_q.shape) == (T, H) and x_q.dtype == FP8 and x_s.dtype == torch.int32
    q_o, b_o = _expect(oracle, x)
    assert torch.equal(x_q.cpu().view(torch.uint8), q_o)
    assert torch.equal(_scale_bytes(x_s, H // 128), b_o)
    if (H // 128) % 4:  # unused bytes of the last word are zero
        words = torch.empty(tuple(x_s.shape), dtype=torch.int32)
        words.copy_(x_s.cpu())
        pad = words.view(torch.uint8).reshape(T, -1)[:, H // 128:]
        assert not bool(pad.any())


def test_fused_matches_unfused_pipeline(gpu, oracle):
    """The other way to write it (the comment at python/sglang/srt/layers/quantization/fp8_kernel.py:335-345): apply the
    activation first, then the ordinary v2 quantizer; same codes and scales when the activation is the same."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8

    x = _data((48, 2 * 1024), torch.bfloat16, 5)
    a_q, a_s = sglang_per_token_group_quant_fp8(
        x.to(gpu), 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True, fuse_silu_and_mul=True, enable_v2=True)
    v = oracle.silu_mul(x)
    b_q, b_s = sglang_per_token_group_quant_fp8(
        v.to(gpu), 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True, enable_v2=True)
    assert torch.equal(a_q.view(torch.uint8), b_q.view(torch.uint8))
    assert torch.equal(_scale_bytes(a_s, 8), _scale_bytes(b_s, 8))


@pytest.mark.parametrize("mode", ["balanced", "imbalanced", "extreme", "empty"])
def test_fused_masked_layout(gpu, oracle, mode):
    from sglang_amd.fp8_kernel import per_token_group_quant_8bit

    E, T, H = 6, 96, 2048
    masked = {"balanced": [40] * E, "imbalanced": [96, 0, 1, 17, 95, 3], "extreme": [77, 0, 0, 0, 0, 0], "empty": [0] * E}[mode]
    x = _data((E, T, 2 * H), torch.bfloat16, 77)
    masked_m = torch.tensor(masked, dtype=torch.int32, device=gpu)
    x_q, x_s = per_token_group_quant_8bit(
        x.to(gpu), 128, FP8, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True, fuse_silu_and_mul=True,
        masked_m=masked_m)
    assert tuple(x_q.shape) == (E, T, H) and tuple(x_s.shape) == (E, T, 4)
    for e in range(E):
        m = masked[e]
        q_e = x_q[e].cpu().view(torch.uint8)
        b_e = _scale_bytes(x_s[e], H // 128)
        if m:
            q_o, b_o = _expect(oracle, x[e, :m].contiguous())
            assert torch.equal(q_e[:m], q_o), (mode, e)
            assert torch.equal(b_e[:m], b_o), (mode, e)
        # rows past masked_m are not written: the wrapper's zeros survive
        assert not bool(q_e[m:].any()) and not bool(b_e[m:].any()), (mode, e)


def test_unsupported_combinations_raise(gpu):
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8

    x = torch.zeros(4, 512, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(NotImplementedError):  # fused, but fp32 scales
        sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True, fuse_silu_and_mul=True, enable_v2=True)
    with pytest.raises(NotImplementedError):  # masked without the fused activation
        sglang_per_token_group_quant_fp8(x, 128, masked_m=torch.zeros(1, dtype=torch.int32, device=gpu), enable_v2=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_every_gate_value(gpu, oracle, dtype):
    """The kernel looks T(silu(gate)) up in a table computed at build time: every one of the 65536 gate bit patterns of
    either input type (infinities and NaNs aside) must give the oracle's value.  With up = 1 the quantized value is
    T(silu(gate)) itself; with up = -3 the product's rounding is exercised too."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8

    T, H = 512, 128
    gate = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype).clone()
    gate[~torch.isfinite(gate.float())] = 0
    for up in (1.0, -3.0):
        x = torch.empty(T, 2 * H, dtype=dtype)
        x[:, :H] = gate.view(T, H)
        x[:, H:] = up
        q, s = sglang_per_token_group_quant_fp8(x.to(gpu), 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True,
                                                fuse_silu_and_mul=True, enable_v2=True)
        v = oracle.silu_mul(x)
        q_o, s_o = oracle.group_quant(v, 128, mode="mul", layout="ue8m0")
        assert torch.equal(q.cpu().view(torch.uint8), q_o.view(torch.uint8))
        dense = torch.empty(tuple(s.shape), dtype=torch.int32)
        dense.copy_(s.cpu())
        assert torch.equal(dense.view(torch.uint8).reshape(T, -1)[:, :1], oracle.unpack_ue8m0(s_o, 1))
