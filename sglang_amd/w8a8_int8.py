"""Forward pass of the INT8 linear method (python/sglang/srt/layers/quantization/w8a8_int8.py:387-417) on the gfx950
kernels: per-token activation quantization, then the INT8 GEMM with the per-token and per-channel scales and the bias
applied in its epilogue."""
from __future__ import annotations

from typing import Optional

import torch

from . import ops
from .int8_kernel import per_token_quant_int8
from .sgl_kernel import int8_scaled_mm


def apply_w8a8_int8_linear(
    x: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor, bias: Optional[torch.Tensor] = None
) -> torch.Tensor:
    """`weight` [K, N] int8, column-major (the checkpoint's [N, K] tensor transposed once at load time,
    w8a8_int8.py:353); `weight_scale` N fp32 values; `x` [..., K]."""
    K, N = weight.shape
    x2d = x.reshape(-1, K)
    if not x2d.is_contiguous():
        x2d = x2d.contiguous()
    w_scale = weight_scale.reshape(-1)
    one_call = (x2d.is_cuda and x2d.shape[0] > 0 and x.dtype in (torch.bfloat16, torch.float16) and weight.dtype == torch.int8
                and weight.stride(0) == 1 and K % 16 == 0 and N % 8 == 0 and w_scale.dtype == torch.float32
                and w_scale.is_contiguous() and w_scale.numel() == N
                and (bias is None or (bias.dtype == x.dtype and bias.is_contiguous() and bias.numel() == N)))
    if one_call:  # the same two kernels on the same data behind one C-ABI call: half the host time, one workspace
        out = ops.int8_linear(x2d, weight, w_scale, bias, x.dtype)
    else:  # anything else goes through the two operators, which raise the reference's errors
        q, s = per_token_quant_int8(x2d)
        out = int8_scaled_mm(q, weight, s, w_scale, out_dtype=x.dtype, bias=bias)
    return out.view(*x.shape[:-1], N)
