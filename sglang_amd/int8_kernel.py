"""The part of ``sglang.srt.layers.quantization.int8_kernel`` used by the INT8 linear
(python/sglang/srt/layers/quantization/w8a8_int8.py:387-417), on the gfx950 kernels."""
from __future__ import annotations

import torch

from . import ops
from .fp8_kernel import sglang_per_token_group_quant_int8  # noqa: F401  (same module in the reference)


def per_token_quant_int8(x: torch.Tensor, scale_dtype: torch.dtype = torch.float32, cal_sum: bool = False):
    """int8_kernel.py:59-89: per-row symmetric quantization, returns ``(x_q, scales[..., 1])`` and, with `cal_sum`, the row
    sums ``x_sum[...]`` in the input's type (fp32 accumulation; the INT8 mixture-of-experts path asks for them)."""
    assert x.is_contiguous()
    assert scale_dtype == torch.float32
    K = x.shape[-1]
    M = x.numel() // K
    x_q = torch.empty_like(x, device=x.device, dtype=torch.int8)
    scales = torch.empty(x.shape[:-1] + (1,), device=x.device, dtype=scale_dtype)
    x_sum = torch.empty(x.shape[:-1], device=x.device, dtype=x.dtype) if cal_sum else None
    ops.per_token_quant_int8(x.view(M, K), x_q, scales, x_sum)
    return (x_q, scales, x_sum) if cal_sum else (x_q, scales)
