"""Forward pass of the INT8 linear method (python/sglang/srt/layers/quantization/w8a8_int8.py:387-417) on the gfx950
kernels: per-token activation quantization, then the INT8 GEMM with the per-token and per-channel scales and the bias
applied in its epilogue."""
from __future__ import annotations

from typing import Optional

import torch

from .int8_kernel import per_token_quant_int8
from .sgl_kernel import int8_scaled_mm


def apply_w8a8_int8_linear(
    x: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor, bias: Optional[torch.Tensor] = None
) -> torch.Tensor:
    """`weight` [K, N] int8, column-major (the checkpoint's [N, K] tensor transposed once at load time,
    w8a8_int8.py:353); `weight_scale` N fp32 values; `x` [..., K]."""
    K, N = weight.shape
    x2d = x.reshape(-1, K)
    q, s = per_token_quant_int8(x2d if x2d.is_contiguous() else x2d.contiguous())
    out = int8_scaled_mm(q, weight, s, weight_scale.reshape(-1), out_dtype=x.dtype, bias=bias)
    return out.view(*x.shape[:-1], N)
