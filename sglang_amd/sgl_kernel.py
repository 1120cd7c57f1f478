"""Python wrappers with the names, arguments and defaults of ``sgl_kernel`` for this path
(sgl-kernel/python/sgl_kernel/gemm.py:14-43, :101-161).  Each goes through
``torch.ops.sgl_kernel.<op>.default`` exactly like the reference's wrappers do."""
from __future__ import annotations

import os
from typing import Optional

import torch

from . import ops

ops.register()


def _get_bool_env_var(name: str, default: str = "false") -> bool:
    # same truth values as sglang.srt.utils.get_bool_env_var
    return os.getenv(name, default).lower() in ("true", "1")


def int8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None):
    return torch.ops.sgl_kernel.int8_scaled_mm.default(mat_a, mat_b, scales_a, scales_b, out_dtype, bias)


def fp8_blockwise_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype):
    return torch.ops.sgl_kernel.fp8_blockwise_scaled_mm.default(mat_a, mat_b, scales_a, scales_b, out_dtype)


def fp8_blockwise_scaled_grouped_mm(output, a_ptrs, b_ptrs, out_ptrs, a_scales_ptrs, b_scales_ptrs, a, b, scales_a, scales_b,
                                    stride_a, stride_b, stride_c, layout_sfa, layout_sfb, problem_sizes, expert_offsets,
                                    workspace):
    """sgl-kernel/python/sgl_kernel/moe.py:96-135."""
    torch.ops.sgl_kernel.fp8_blockwise_scaled_grouped_mm.default(
        output, a_ptrs, b_ptrs, out_ptrs, a_scales_ptrs, b_scales_ptrs, a, b, scales_a, scales_b, stride_a, stride_b,
        stride_c, layout_sfa, layout_sfb, problem_sizes, expert_offsets, workspace)


def es_fp8_blockwise_scaled_grouped_mm(output, a, b, scales_a, scales_b, stride_a, stride_b, stride_d, problem_sizes,
                                       expert_offsets, workspace):
    """sgl-kernel/python/sgl_kernel/expert_specialization.py:4-28."""
    torch.ops.sgl_kernel.es_fp8_blockwise_scaled_grouped_mm.default(
        output, a, b, scales_a, scales_b, stride_a, stride_b, stride_d, problem_sizes, expert_offsets, workspace)


def fp8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None):
    return torch.ops.sgl_kernel.fp8_scaled_mm.default(mat_a, mat_b, scales_a, scales_b, out_dtype, bias)


def sgl_per_token_quant_fp8(input: torch.Tensor, output_q: torch.Tensor, output_s: torch.Tensor) -> None:
    torch.ops.sgl_kernel.sgl_per_token_quant_fp8.default(input, output_q, output_s)


def sgl_per_tensor_quant_fp8(input: torch.Tensor, output_q: torch.Tensor, output_s: torch.Tensor, is_static: bool) -> None:
    """sgl-kernel/python/sgl_kernel/gemm.py:145-153."""
    torch.ops.sgl_kernel.sgl_per_tensor_quant_fp8.default(input, output_q, output_s, is_static)


def sgl_per_token_group_quant_8bit(
    input: torch.Tensor,
    output_q: torch.Tensor,
    output_s: torch.Tensor,
    group_size: int,
    eps: float,
    fp8_min: float,
    fp8_max: float,
    scale_ue8m0: bool = False,
    fuse_silu_and_mul: bool = False,
    masked_m: Optional[torch.Tensor] = None,
    enable_v2: Optional[bool] = None,
) -> None:
    if enable_v2 is None:
        enable_v2 = _get_bool_env_var("SGLANG_PER_TOKEN_GROUP_QUANT_8BIT_V2")

    if enable_v2:
        return torch.ops.sgl_kernel.sgl_per_token_group_quant_8bit_v2.default(
            input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0, fuse_silu_and_mul, masked_m
        )

    assert not fuse_silu_and_mul, "only v2 support fuse_silu_and_mul"
    assert masked_m is None, "only v2 support masked_m"
    torch.ops.sgl_kernel.sgl_per_token_group_quant_8bit.default(
        input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0
    )


# legacy names kept by the reference
sgl_per_token_group_quant_fp8 = sgl_per_token_group_quant_8bit
sgl_per_token_group_quant_int8 = sgl_per_token_group_quant_8bit
