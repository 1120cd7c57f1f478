"""Seeded synthetic inputs for the quantized-linear path.

Everything is generated on the CPU with an explicit ``torch.Generator`` so that the CPU
checker and the GPU kernels see identical bits; callers copy to the device afterwards.
Only plain torch is used here.

The shapes and distributions are the ones the reference's own tests and benchmarks use:
  * activations: ``sgl-kernel/python/sgl_kernel/test_utils.py:4-62`` (bf16 randn with a
    fraction of amplified elements, seed ``num_tokens * 10000 + hidden_dim``);
  * block-quantized fp8 weights: ``python/sglang/test/test_block_fp8_deep_gemm_blackwell.py:22-45``
    (per 128x128 block ``amax`` clamped at 1e-4, ``scale = amax / 448``, ``q = w * (448 / amax)``);
  * int8 operands: ``python/sglang/srt/layers/quantization/int8_kernel.py:47-50`` for the
    activation, symmetric per-output-channel for the weight.
"""
from __future__ import annotations

from typing import Tuple

import torch

FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0

# (K, N) of the linear layers the benchmark configurations name.
DSV3_MLP = {"gate_up": (7168, 36864), "down": (18432, 7168)}
DSV3_MLA = {"q_a": (7168, 1536), "kv_a": (7168, 576), "q_b": (1536, 24576), "kv_b": (512, 32768)}
LLAMA3_8B = {"qkv": (4096, 6144), "gate_up": (4096, 28672), "down": (14336, 4096)}


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(int(seed))
    return g


def cdiv(a: int, b: int) -> int:
    return -(-a // b)


def make_activation(
    M: int,
    K: int,
    seed: int | None = None,
    dtype: torch.dtype = torch.bfloat16,
    outlier_frac: float = 1e-3,
    outlier_gain: float = 50.0,
    zero_group_frac: float = 0.0,
    zero_elem_frac: float = 0.0,
    group: int = 128,
) -> torch.Tensor:
    """N(0,1) activations with a Bernoulli(outlier_frac) mask of elements multiplied by
    ``outlier_gain``; optionally whole groups and single elements forced to zero so that
    some groups have amax == 0."""
    g = _gen(M * 10000 + K if seed is None else seed)
    x = torch.randn(M, K, generator=g, dtype=torch.float32)
    if outlier_frac > 0:
        mask = torch.rand(M, K, generator=g) < outlier_frac
        x = torch.where(mask, x * outlier_gain, x)
    if zero_elem_frac > 0:
        x = torch.where(torch.rand(M, K, generator=g) < zero_elem_frac, torch.zeros(()), x)
    if zero_group_frac > 0:
        zg = torch.rand(M, K // group, generator=g) < zero_group_frac
        x = x.view(M, K // group, group).masked_fill(zg[..., None], 0.0).view(M, K)
    return x.to(dtype).contiguous()


def block_cast_to_fp8(w: torch.Tensor, block: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """[N, K] fp32 -> (fp8 [N, K], fp32 scales [ceil(N/b), ceil(K/b)]), one scale per block."""
    N, K = w.shape
    Np, Kp = cdiv(N, block) * block, cdiv(K, block) * block
    wp = torch.zeros(Np, Kp, dtype=torch.float32)
    wp[:N, :K] = w
    v = wp.view(Np // block, block, Kp // block, block)
    amax = v.abs().amax(dim=(1, 3), keepdim=True).clamp(min=1e-4)
    q = (v * (FP8_MAX / amax)).clamp(-FP8_MAX, FP8_MAX).to(FP8)
    q = q.view(Np, Kp)[:N, :K].contiguous()
    s = (amax / FP8_MAX).view(Np // block, Kp // block).contiguous()
    return q, s


def make_fp8_weight(N: int, K: int, seed: int | None = None, std: float = 0.02):
    """N(0, std) weights quantized per 128x128 block: (fp8 [N,K], fp32 [ceil(N/128), ceil(K/128)])."""
    g = _gen(N * 10007 + K if seed is None else seed)
    w = torch.randn(N, K, generator=g, dtype=torch.float32) * std
    return block_cast_to_fp8(w)


def make_int8_activation(M: int, K: int, seed: int | None = None):
    """bf16 N(0,1) activations quantized per token: (int8 [M,K], fp32 scales [M,1])."""
    g = _gen(M * 10000 + K + 1 if seed is None else seed)
    x = torch.randn(M, K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(torch.float32)
    amax = x.abs().amax(dim=1, keepdim=True).clamp(min=1e-10)
    t = x * (127.0 / amax)
    q = (torch.sign(t) * torch.floor(t.abs() + 0.5)).to(torch.int8)
    return q.contiguous(), (amax / 127.0).contiguous()


def make_int8_weight(N: int, K: int, seed: int | None = None, std: float = 0.02):
    """N(0, std) weights, symmetric per output channel: (int8 [N,K], fp32 scales [N])."""
    g = _gen(N * 10009 + K if seed is None else seed)
    w = torch.randn(N, K, generator=g, dtype=torch.float32) * std
    amax = w.abs().amax(dim=1, keepdim=True).clamp(min=1e-10)
    s = amax / 127.0
    q = torch.round(w / s).clamp(-127, 127).to(torch.int8)
    return q.contiguous(), s.view(-1).contiguous()


def quant_algorithmic_bytes(M: int, K: int, group: int, in_bytes: int = 2, ue8m0: bool = False) -> int:
    """Bytes the group quantizer must move: read x, write q, write one scale per group."""
    groups = M * (K // group)
    return M * K * in_bytes + M * K + groups * (1 if ue8m0 else 4)


def gemm_flops(M: int, N: int, K: int) -> int:
    return 2 * M * N * K


def fp8_gemm_algorithmic_bytes(M: int, N: int, K: int, out_bytes: int = 2) -> int:
    """Weight-streaming bytes of one blockwise-FP8 linear: W, A, both scale sets, output."""
    return N * K + M * K + 4 * M * cdiv(K, 128) + 4 * cdiv(N, 128) * cdiv(K, 128) + out_bytes * M * N


def int8_gemm_algorithmic_bytes(M: int, N: int, K: int, out_bytes: int = 2) -> int:
    return N * K + M * K + 4 * M + 4 * N + out_bytes * M * N
