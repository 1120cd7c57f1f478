"""The INT8 linear method's forward (python/sglang/srt/layers/quantization/w8a8_int8.py:387-417) on the gfx950 kernels."""
from __future__ import annotations

from typing import Optional

import torch

from .int8_kernel import per_token_quant_int8
from .sgl_kernel import int8_scaled_mm


def apply_w8a8_int8_linear(
    x: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor, bias: Optional[torch.Tensor] = None
) -> torch.Tensor:
    """`weight` is the layer's int8 weight as the reference keeps it after loading: shape [K, N], column-major
    (`weight.t()` of the [N, K] checkpoint tensor, w8a8_int8.py:353); `weight_scale` [N, 1] fp32."""
    x_q, x_scale = per_token_quant_int8(x)

    x_q_2d = x_q.view(-1, x_q.shape[-1])
    x_scale_2d = x_scale.view(-1, x_scale.shape[-1])
    output_shape = [*x_q.shape[:-1], weight.shape[1]]

    output = int8_scaled_mm(x_q_2d, weight, x_scale_2d, weight_scale, out_dtype=x.dtype, bias=bias)
    return output.view(output_shape)
