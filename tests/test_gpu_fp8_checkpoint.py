"""GPU side of FP8 checkpoint ingestion: layers built by sglang_amd.fp8 from checkpoint tensors run the gfx950 kernels and
agree with the CPU oracle applied to the same checkpoint tensors (quantizer bit-exact, GEMM within
|out - ref| <= 1e-2 * |ref| + 1e-4 * mag, the criterion of tests/fp8_tolerance.py).
Tensor-parallel shards are run one after the other on the one GPU: column-parallel outputs are concatenated, row-parallel
partial sums are added in fp32 (the caller's all-reduce)."""
import pytest
import torch

from fp8_tolerance import check_fp8_gemm
from sglang_amd.workloads import make_activation

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
BLOCK_CFG = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic", "weight_block_size": [128, 128]}


def _proj(n, k, g, name):
    w = ((torch.rand(n, k, generator=g) - 0.5) * 896).clamp(-448, 448).to(FP8)
    s = torch.rand((n + 127) // 128, (k + 127) // 128, generator=g) * 1e-3 + 1e-4
    return {f"{name}.weight": w, f"{name}.weight_scale_inv": s}


def _close(out, ref, mag, extra=0.0):
    check_fp8_gemm(out, ref, mag, extra=extra)


@pytest.mark.parametrize("M", [3, 200])
def test_block_fp8_merged_layer_and_its_shards(gpu, oracle, M):
    from sglang_amd.fp8 import Fp8Config, Fp8Linear

    cfg = Fp8Config.from_config(BLOCK_CFG)
    g = torch.Generator().manual_seed(4)
    K, N1 = 1024, 768
    ckpt = {**_proj(N1, K, g, "gate_proj"), **_proj(N1, K, g, "up_proj"), **_proj(K, N1, g, "down_proj")}
    x = make_activation(M, K, seed=M)
    x_q, x_s = oracle.group_quant(x, 128, mode="div", layout="row")
    w_full = torch.cat([ckpt["gate_proj.weight"], ckpt["up_proj.weight"]])
    s_full = torch.cat([ckpt["gate_proj.weight_scale_inv"], ckpt["up_proj.weight_scale_inv"]])
    ref, mag = oracle.fp8_blockwise_mm(x_q, w_full, x_s, s_full, torch.float32, want_abs=True)

    layer = Fp8Linear(K, [N1, N1], cfg, device=gpu)
    layer.load_from(ckpt, ["gate_proj", "up_proj"])
    layer.process_weights_after_loading()
    out = layer(x.to(gpu).view(1, M, K))
    assert tuple(out.shape) == (1, M, 2 * N1) and out.dtype == torch.bfloat16
    _close(out.view(M, -1), ref, mag)

    # column-parallel over 3 ranks: rank r holds channels [r*256, +256) of gate and of up
    outs = []
    for r in range(3):
        part = Fp8Linear(K, [N1, N1], cfg, parallel="column", tp_rank=r, tp_size=3, device=gpu)
        part.load_from(ckpt, ["gate_proj", "up_proj"])
        part.process_weights_after_loading()
        outs.append(part(x.to(gpu)))
    gate = torch.cat([o[:, :256] for o in outs], dim=1)
    up = torch.cat([o[:, 256:] for o in outs], dim=1)
    _close(torch.cat([gate, up], dim=1), ref, mag)

    # row-parallel down projection over 2 ranks: each rank quantizes and multiplies its own K slice
    h = make_activation(M, N1, seed=50 + M)
    h_q, h_s = oracle.group_quant(h, 128, mode="div", layout="row")
    ref_d, mag_d = oracle.fp8_blockwise_mm(h_q, ckpt["down_proj.weight"], h_s, ckpt["down_proj.weight_scale_inv"], torch.float32,
                                           want_abs=True)
    total = torch.zeros(M, K)
    for r in range(2):
        part = Fp8Linear(N1, [K], cfg, parallel="row", tp_rank=r, tp_size=2, device=gpu)
        part.load_from(ckpt, ["down_proj"])
        part.process_weights_after_loading()
        total += part(h.to(gpu)[:, r * (N1 // 2):(r + 1) * (N1 // 2)].contiguous()).float().cpu()
    _close(total, ref_d, mag_d, extra=2.0 ** -7 * mag_d.clamp(max=ref_d.abs().max()))  # two bf16-rounded partial sums


def test_requantized_to_power_of_two_scales(gpu, oracle):
    """process_weights_after_loading(requant_ue8m0=True): the layer then holds packed exponents and runs the GEMM whose
    scales the MFMA applies; the result is the oracle's on the re-quantized weight (oracle.block_dequant / block_cast)."""
    from sglang_amd.fp8 import Fp8Config, Fp8Linear

    cfg = Fp8Config.from_config(BLOCK_CFG)
    g = torch.Generator().manual_seed(6)
    K, N, M = 512, 640, 64
    ckpt = _proj(N, K, g, "o_proj")
    layer = Fp8Linear(K, [N], cfg, device=gpu, bias=True)
    ckpt["o_proj.bias"] = torch.randn(N, generator=g).to(torch.bfloat16)
    layer.load_from(ckpt, ["o_proj"])
    layer.process_weights_after_loading(requant_ue8m0=True)
    assert layer.weight_scale_inv.dtype == torch.int32 and tuple(layer.weight_scale_inv.shape) == (N, 1)
    x = make_activation(M, K, seed=8)
    out = layer(x.to(gpu))
    w2, s2 = oracle.block_cast_to_fp8(oracle.block_dequant_fp8(ckpt["o_proj.weight"], ckpt["o_proj.weight_scale_inv"]))
    assert torch.equal(layer.weight.data.cpu().view(torch.uint8), w2.view(torch.uint8))
    x_q, x_s = oracle.group_quant(x, 128, mode="mul", layout="ue8m0")
    sa = torch.ldexp(torch.ones(M, K // 128), oracle.unpack_ue8m0(x_s, K // 128).to(torch.int32) - 127)
    ref, mag = oracle.fp8_blockwise_mm(x_q, w2, sa, s2, torch.float32, want_abs=True)
    # the linear rounds the product to bf16 and then adds the bias, as the reference's wrappers do: up to half a unit in the last place of the product, 2^-8 of it
    _close(out, ref + ckpt["o_proj.bias"].float()[None, :], mag, extra=2.0 ** -8 * ref.abs())


def test_per_tensor_static_checkpoint(gpu, oracle):
    from sglang_amd.fp8 import Fp8Config, Fp8Linear

    cfg = Fp8Config.from_config({"quant_method": "fp8", "activation_scheme": "static"})
    g = torch.Generator().manual_seed(7)
    K, sizes, M = 512, [256, 128, 128], 37
    layer = Fp8Linear(K, sizes, cfg, device=gpu)
    tensors, ws = {}, [0.004, 0.002, 0.003]
    x = make_activation(M, K, seed=9)
    in_scale = float(x.float().abs().max()) / 300.0
    for name, n, s in zip("qkv", sizes, ws):
        tensors[f"{name}.weight"] = ((torch.rand(n, K, generator=g) - 0.5) * 896).clamp(-448, 448).to(FP8)
        tensors[f"{name}.weight_scale"] = torch.tensor(s)
        tensors[f"{name}.input_scale"] = torch.tensor(in_scale * (0.5 if name == "k" else 1.0))
    layer.load_from(tensors, ["q", "k", "v"])
    layer.process_weights_after_loading()
    out = layer(x.to(gpu))
    scale = torch.tensor([in_scale], dtype=torch.float32)
    q_o, _ = oracle.per_tensor_quant_fp8(x, scale)
    w = torch.cat([tensors[f"{n}.weight"] for n in "qkv"])
    sb = torch.cat([torch.full((n,), s) for n, s in zip(sizes, ws)])
    ref, mag = oracle.fp8_scaled_mm(q_o, w, scale.expand(M).contiguous(), sb, torch.float32, None, want_abs=True)
    _close(out, ref, mag)


@pytest.mark.parametrize("K,sizes", [(7168, [256, 128]), (1024, [384])])
def test_sixteen_bit_checkpoint_is_quantized_per_channel_at_load(gpu, oracle, K, sizes):
    """fp8.py:368-383: a bf16 checkpoint under quantization="fp8": one quantization group per output channel
    (per_token_group_quant_fp8 with group_size = K), dynamic per-token activations, fp8_scaled_mm."""
    from sglang_amd.fp8 import Fp8Config, Fp8Linear

    cfg = Fp8Config.from_config({"quant_method": "none", "activation_scheme": "dynamic"})
    assert not cfg.is_checkpoint_fp8_serialized
    g = torch.Generator().manual_seed(3)
    M = 19
    layer = Fp8Linear(K, sizes, cfg, device=gpu)
    names = ["gate", "up"][:len(sizes)]
    tensors = {f"{n}.weight": (torch.randn(sz, K, generator=g) * 0.02).to(torch.bfloat16) for n, sz in zip(names, sizes)}
    layer.load_from(tensors, names)
    layer.process_weights_after_loading()
    w16 = torch.cat([tensors[f"{n}.weight"] for n in names])
    wq_o, ws_o = oracle.group_quant(w16, K, mode="rcp", layout="row")
    assert tuple(layer.weight.shape) == (K, sum(sizes)) and tuple(layer.weight_scale.shape) == (1, sum(sizes))
    assert torch.equal(layer.weight.data.t().contiguous().cpu().view(torch.uint8), wq_o.view(torch.uint8))
    assert torch.equal(layer.weight_scale.data.cpu().view(-1), ws_o.view(-1))
    x = make_activation(M, K, seed=5)
    out = layer(x.to(gpu))
    q_o, s_o = oracle.per_token_quant_fp8(x)
    ref, mag = oracle.fp8_scaled_mm(q_o, wq_o, s_o.view(-1), ws_o.view(-1), torch.float32, None, want_abs=True)
    _close(out, ref, mag)
