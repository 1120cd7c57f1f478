"""GPU parity of the per-tensor FP8 quantizer (sgl_per_tensor_quant_fp8, static_quant_fp8, scaled_fp8_quant): codes and
the scale bit-exact against the oracle; and of apply_fp8_linear's static and compressed-tensor paths, which feed
fp8_scaled_mm (|out - ref| <= 1e-2 * |ref| + 1e-4 * mag as in tests/test_gpu_per_token_fp8.py)."""
import pytest
import torch

from fp8_tolerance import check_fp8_gemm
from sglang_amd.workloads import make_activation

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def _bits(t):
    return t.cpu().view(torch.uint8)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M,K", [(1, 8), (3, 1000), (64, 7168), (1, 5), (1024, 4096), (7, 16384 + 24)])
def test_dynamic_bits(gpu, oracle, dtype, M, K):
    from sglang_amd.sgl_kernel import sgl_per_tensor_quant_fp8

    x = make_activation(M, K, seed=3 * M + K, dtype=dtype)
    xg = x.to(gpu)
    q = torch.empty(M, K, dtype=FP8, device=gpu)
    s = torch.zeros(1, dtype=torch.float32, device=gpu)
    sgl_per_tensor_quant_fp8(xg, q, s, False)
    q_o, s_o = oracle.per_tensor_quant_fp8(x)
    assert torch.equal(s.cpu().view(torch.int32), s_o.view(torch.int32))
    assert torch.equal(_bits(q), q_o.view(torch.uint8))
    # the same tensor quantized statically with that scale gives the same codes; the scale is left alone
    q2 = torch.empty_like(q)
    s2 = s.clone()
    sgl_per_tensor_quant_fp8(xg, q2, s2, True)
    assert torch.equal(_bits(q2), _bits(q)) and torch.equal(s2, s)


def test_zero_tensor_like_the_reference(gpu, oracle):
    from sglang_amd.sgl_kernel import sgl_per_tensor_quant_fp8

    x = torch.zeros(5, 256, dtype=torch.bfloat16)
    q = torch.empty(5, 256, dtype=FP8, device=gpu)
    s = torch.zeros(1, dtype=torch.float32, device=gpu)
    sgl_per_tensor_quant_fp8(x.to(gpu), q, s, False)
    q_o, s_o = oracle.per_tensor_quant_fp8(x)
    assert float(s) == 0.0 and torch.equal(_bits(q), q_o.view(torch.uint8))


@pytest.mark.parametrize("repeat", [False, True])
def test_static_quant_fp8(gpu, oracle, repeat):
    from sglang_amd.fp8_kernel import static_quant_fp8

    x = make_activation(37, 2048, seed=5)
    scale = torch.tensor([0.0371], dtype=torch.float32)
    q, s = static_quant_fp8(x.to(gpu), scale.to(gpu), repeat_scale=repeat)
    q_o, _ = oracle.per_tensor_quant_fp8(x, scale)
    assert torch.equal(_bits(q), q_o.view(torch.uint8))
    if repeat:
        assert tuple(s.shape) == (37, 1) and bool((s.cpu() == scale).all())
    else:
        assert s.numel() == 1 and float(s) == float(scale)


def test_scaled_fp8_quant_modes(gpu, oracle):
    from sglang_amd.fp8_kernel import scaled_fp8_quant

    x = make_activation(19, 1024, seed=6)
    xg = x.to(gpu)
    q, s = scaled_fp8_quant(xg)  # dynamic per tensor
    q_o, s_o = oracle.per_tensor_quant_fp8(x)
    assert s.numel() == 1 and torch.equal(s.cpu(), s_o) and torch.equal(_bits(q), q_o.view(torch.uint8))
    q, s = scaled_fp8_quant(xg, use_per_token_if_dynamic=True)  # dynamic per token
    q_o, s_o = oracle.per_token_quant_fp8(x)
    assert tuple(s.shape) == (19, 1) and torch.equal(s.cpu(), s_o) and torch.equal(_bits(q), q_o.view(torch.uint8))
    given = torch.tensor([0.02], dtype=torch.float32)
    q, s = scaled_fp8_quant(xg, given.to(gpu), num_token_padding=32)  # static, padded output
    q_o, _ = oracle.per_tensor_quant_fp8(x, given)
    assert tuple(q.shape) == (32, 1024) and torch.equal(_bits(q[:19]), q_o.view(torch.uint8)) and float(s) == float(given)


@pytest.mark.parametrize("path", ["static", "compressed_static", "compressed_dynamic_tensor", "compressed_dynamic_token"])
def test_apply_fp8_linear_paths(gpu, oracle, path):
    from sglang_amd.fp8_utils import apply_fp8_linear

    M, K, N = 45, 1024, 768
    g = torch.Generator().manual_seed(17)
    x = make_activation(M, K, seed=7)
    w = ((torch.rand(N, K, generator=g) - 0.5) * 2 * 448.0).clamp(-448, 448).to(FP8)
    ws = torch.rand(N, generator=g) * 1e-3 + 1e-4
    bias = torch.randn(N, generator=g).to(torch.bfloat16)
    in_scale = torch.tensor([float(x.float().abs().max()) / 300.0], dtype=torch.float32)
    kw = dict(bias=bias.to(gpu))
    if path == "static":
        kw.update(input_scale=in_scale.to(gpu))
        q_o, _ = oracle.per_tensor_quant_fp8(x, in_scale)
        sa = in_scale.expand(M)
    elif path == "compressed_static":
        kw.update(input_scale=in_scale.to(gpu), compressed_tensor_quant=True)
        q_o, _ = oracle.per_tensor_quant_fp8(x, in_scale)
        sa = in_scale.expand(M)
    elif path == "compressed_dynamic_tensor":
        kw.update(compressed_tensor_quant=True)
        q_o, s_o = oracle.per_tensor_quant_fp8(x)
        sa = s_o.expand(M)
    else:
        kw.update(compressed_tensor_quant=True, use_per_token_if_dynamic=True)
        q_o, s_o = oracle.per_token_quant_fp8(x)
        sa = s_o.reshape(M)
    out = apply_fp8_linear(x.to(gpu).view(5, 9, K), w.to(gpu).t(), ws.to(gpu), **kw)
    assert tuple(out.shape) == (5, 9, N) and out.dtype == torch.bfloat16
    ref, mag = oracle.fp8_scaled_mm(q_o, w, sa.contiguous(), ws, torch.float32, None, want_abs=True)
    ref = ref + bias.float()[None, :]
    check_fp8_gemm(out.reshape(M, N), ref, mag, path)
