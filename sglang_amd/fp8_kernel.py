"""The part of ``sglang.srt.layers.quantization.fp8_kernel`` that sits on the quantized-linear
path, with the reference's names, arguments, defaults and return conventions, running on the
gfx950 kernels instead of Triton.

gfx950 uses OCP e4m3fn (max 448), like NVIDIA parts; the reference's HIP branch hard-codes
224 for the older fnuz format (fp8_kernel.py:243-248), which does not apply here.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from . import _lib, ops
from .sgl_kernel import sgl_per_token_group_quant_8bit

fp8_dtype = torch.float8_e4m3fn
fp8_max = torch.finfo(fp8_dtype).max
fp8_min = -fp8_max


def align(x: int, a: int) -> int:
    return (x + a - 1) // a * a


def ceil_div(a: int, b: int) -> int:
    return -(-a // b)


def create_per_token_group_quant_fp8_output_scale(
    x_shape,
    device,
    group_size,
    column_major_scales: bool,
    scale_tma_aligned: bool,
    scale_ue8m0: bool,
):
    """Scale tensor with the shapes and strides of fp8_kernel.py:433-474."""
    x_shape = tuple(x_shape)
    if scale_ue8m0:
        assert column_major_scales and scale_tma_aligned
        *x_batch, x_q_mn, x_q_k = x_shape
        x_s_mn, x_s_k = x_q_mn, x_q_k // 128
        aligned_mn = align(x_s_mn, 4)
        aligned_k = align(x_s_k, 4)
        return torch.empty((*x_batch, aligned_k // 4, aligned_mn), device=device, dtype=torch.int).transpose(-1, -2)[
            ..., :x_s_mn, :
        ]
    elif column_major_scales:
        if scale_tma_aligned:
            aligned_size = (x_shape[-2] + 3) // 4 * 4
            return torch.empty(
                x_shape[:-2] + (x_shape[-1] // group_size, aligned_size), device=device, dtype=torch.float32
            ).transpose(-1, -2)[: x_shape[-2], :]
        else:
            return torch.empty(
                (x_shape[-1] // group_size,) + x_shape[:-1], device=device, dtype=torch.float32
            ).permute(-1, -2)
    else:
        return torch.empty(x_shape[:-1] + (x_shape[-1] // group_size,), device=device, dtype=torch.float32)


def _per_token_group_quant_8bit_raw(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    dtype: torch.dtype = fp8_dtype,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    scale_ue8m0: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp8_kernel.py:215-319.  Row-major scales use ``q = x * (1.0 / s)`` (Triton kernel :155-158),
    column-major scales use ``q = x / s`` (:205-209).  With ``scale_ue8m0`` the reference rounds
    ``s`` up to a power of two and repacks the fp32 scales with DeepGEMM's
    ``transform_sf_into_required_layout``; here the kernel writes that packed int32 layout
    directly (four exponent bytes per word, words column-major and padded to 4 rows)."""
    assert x.shape[-1] % group_size == 0, "the last dimension of `x` cannot be divisible by `group_size`"
    assert x.is_contiguous(), "`x` is not contiguous"

    if dtype == torch.int8:
        bit8_max, bit8_min = 127.0, -128.0
    else:
        info = torch.finfo(dtype)
        bit8_max, bit8_min = info.max, info.min

    x_q = torch.empty_like(x, device=x.device, dtype=dtype)
    if scale_ue8m0:
        assert column_major_scales and group_size == 128
    x_s = create_per_token_group_quant_fp8_output_scale(
        x_shape=x.shape,
        device=x.device,
        group_size=group_size,
        column_major_scales=column_major_scales,
        scale_tma_aligned=scale_tma_aligned or scale_ue8m0,
        scale_ue8m0=scale_ue8m0,
    )
    if x.numel() == 0:
        return x_q, x_s
    K = x.shape[-1]
    M = x.numel() // K
    if column_major_scales:
        assert x_s.dim() == 2, "column-major scales are defined for 2-D inputs"
        mode, s_row, s_col = _lib.QUANT_DIV, 1, x_s.stride(1)
    else:
        assert not scale_ue8m0
        mode, s_row, s_col = _lib.QUANT_RCP, K // group_size, 1
    if (group_size == K and dtype == fp8_dtype and not scale_ue8m0
            and (group_size * x.element_size() > 2048 or group_size & (group_size - 1))):
        # the whole row is one group (a weight quantized per output channel at load time, fp8.py:368-375): rows
        # longer than the group kernel's 2048 bytes, or not a power of two
        _lib.check(_lib.lib().mi355_row_group_quant_fp8(x.data_ptr(), ops._DT[x.dtype], x_q.data_ptr(), x_s.data_ptr(), M, K, eps,
                                                        mode, torch.cuda.current_stream().cuda_stream))
        return x_q, x_s
    kind = _lib.SCALE_UE8M0_PACKED if scale_ue8m0 else _lib.SCALE_F32
    _lib.check(
        _lib.lib().mi355_group_quant_8bit(
            x.data_ptr(), ops._DT[x.dtype], x_q.data_ptr(), ops._DT[dtype], x_s.data_ptr(), M, K, group_size,
            eps, bit8_min, bit8_max, mode, kind, 0.0, s_row, s_col, torch.cuda.current_stream().cuda_stream,
        )
    )
    return x_q, x_s


# backward compatibility (fp8_kernel.py:323)
per_token_group_quant_fp8 = _per_token_group_quant_8bit_raw


def _per_token_group_quant_8bit_fuse_silu_and_mul(
    x: torch.Tensor,
    group_size: int,
    dst_dtype: torch.dtype,
    column_major_scales: bool,
    scale_tma_aligned: bool,
    scale_ue8m0: bool,
    masked_m: Optional[torch.Tensor],
) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp8_kernel.py:325-397: silu(gate) * up, then the 1x128 quantizer with packed UE8M0 scales; ``x`` is [T, 2H] or,
    with ``masked_m``, [E, T, 2H].  The reference goes through a Triton kernel and DeepGEMM's layout transform; its own
    test holds that pair equal to the fused v2 kernel, which is what runs here.  Outputs start as zeros, as there
    (rows past ``masked_m`` stay zero)."""
    assert column_major_scales
    assert scale_tma_aligned
    assert scale_ue8m0
    assert group_size == 128
    out_shape = (*x.shape[:-1], x.shape[-1] // 2)
    output = torch.zeros(out_shape, device=x.device, dtype=dst_dtype)
    output_scale = create_per_token_group_quant_fp8_output_scale(
        x_shape=out_shape, device=x.device, group_size=group_size, column_major_scales=True, scale_tma_aligned=True,
        scale_ue8m0=True,
    )
    output_scale.zero_()
    if x.numel() > 0:
        sgl_per_token_group_quant_8bit(
            x, output, output_scale, group_size, 1e-10, fp8_min, fp8_max, True, True, masked_m, enable_v2=True,
        )
    return output, output_scale


def per_token_group_quant_8bit(
    x: torch.Tensor,
    group_size: int,
    dst_dtype: torch.dtype,
    eps: float = 1e-10,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    scale_ue8m0: bool = False,
    fuse_silu_and_mul: bool = False,
    masked_m: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp8_kernel.py:400-430."""
    if fuse_silu_and_mul:
        return _per_token_group_quant_8bit_fuse_silu_and_mul(
            x=x, group_size=group_size, dst_dtype=dst_dtype, column_major_scales=column_major_scales,
            scale_tma_aligned=scale_tma_aligned, scale_ue8m0=scale_ue8m0, masked_m=masked_m,
        )
    if masked_m is not None:
        raise NotImplementedError("masked_m without fuse_silu_and_mul has no kernel in the reference either")
    return _per_token_group_quant_8bit_raw(
        x=x,
        group_size=group_size,
        eps=eps,
        column_major_scales=column_major_scales,
        scale_tma_aligned=scale_tma_aligned,
        scale_ue8m0=scale_ue8m0,
        dtype=dst_dtype,
    )


def sglang_per_token_group_quant_fp8(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    scale_ue8m0: bool = False,
    fuse_silu_and_mul: bool = False,
    masked_m: Optional[torch.Tensor] = None,
    enable_v2: Optional[bool] = None,
):
    """fp8_kernel.py:477-527: allocate outputs, then ``sgl_per_token_group_quant_8bit``."""
    assert x.shape[-1] % group_size == 0, "the last dimension of `x` cannot be divisible by `group_size`"
    assert x.is_contiguous(), "`x` is not contiguous"

    out_shape = (*x.shape[:-1], x.shape[-1] // (2 if fuse_silu_and_mul else 1))

    x_q = torch.empty(out_shape, device=x.device, dtype=fp8_dtype)
    x_s = create_per_token_group_quant_fp8_output_scale(
        x_shape=out_shape,
        device=x.device,
        group_size=group_size,
        column_major_scales=column_major_scales,
        scale_tma_aligned=scale_tma_aligned,
        scale_ue8m0=scale_ue8m0,
    )

    if x.shape[0] > 0:
        sgl_per_token_group_quant_8bit(
            x, x_q, x_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0, fuse_silu_and_mul, masked_m,
            enable_v2=enable_v2,
        )

    return x_q, x_s


def w8a8_block_fp8_matmul_deepgemm(A: torch.Tensor, B: torch.Tensor, As: torch.Tensor, Bs: torch.Tensor,
                                   block_size: List[int], output_dtype: torch.dtype) -> torch.Tensor:
    """fp8_kernel.py:1047-1065: C = A @ B^T with packed UE8M0 scales on both operands (DeepGEMM's gemm_nt_f8f8bf16 in
    the reference): ``As`` int32 [..., M, ceil(K/512)] packed along tokens, ``Bs`` int32 [N, ceil(K/512)] packed along
    weight rows (fp8_utils.transform_scale_ue8m0)."""
    assert list(block_size) == [128, 128]
    assert output_dtype == torch.bfloat16, "Deepgemm only supports output tensor type as bfloat16"
    K = A.shape[-1]
    a2 = A.reshape(-1, K)
    as2 = As.reshape(-1, As.shape[-1]) if As.dim() > 2 else As
    C = ops.fp8_blockwise_mm_ue8m0(a2, B, as2, Bs, output_dtype)
    return C.view(*A.shape[:-1], B.shape[0])


def sglang_per_token_quant_fp8(x: torch.Tensor, dtype: torch.dtype = fp8_dtype):
    """fp8_kernel.py:573-589: one scale per row, ``(x_q, x_s [M, 1])``."""
    assert x.is_contiguous(), "`x` is not contiguous"
    x_q = torch.empty_like(x, device=x.device, dtype=dtype)
    x_s = torch.empty(x.shape[0], 1, device=x.device, dtype=torch.float32)
    from .sgl_kernel import sgl_per_token_quant_fp8

    sgl_per_token_quant_fp8(x, x_q, x_s)
    return x_q, x_s


def static_quant_fp8(x: torch.Tensor, x_s: torch.Tensor, repeat_scale: bool = False):
    """fp8_kernel.py:635-665: quantize with a given per-tensor scale; with ``repeat_scale`` the returned scale is a
    ``[M, 1]`` tensor holding it once per row (the shape fp8_scaled_mm takes)."""
    assert x.is_contiguous(), "`x` is not contiguous"
    assert x_s.numel() == 1, "only supports per-tensor scale"
    x_q = torch.empty_like(x, device=x.device, dtype=fp8_dtype)
    scale = x_s.reshape(1).to(torch.float32)
    if repeat_scale:
        M = x.numel() // x.shape[-1]
        x_s_repeat = torch.empty((M, 1), device=x.device, dtype=torch.float32)
        ops.static_quant_fp8_repeat(x, x_q, scale, x_s_repeat)
        return x_q, x_s_repeat
    from .sgl_kernel import sgl_per_tensor_quant_fp8

    sgl_per_tensor_quant_fp8(x, x_q, scale, True)
    return x_q, x_s


def scaled_fp8_quant(
    input: torch.Tensor,
    scale: Optional[torch.Tensor] = None,
    num_token_padding: Optional[int] = None,
    use_per_token_if_dynamic: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp8_kernel.py:1429-1463: dynamic per-tensor (scale None), dynamic per-token, or static per-tensor quantization.
    Rows added by ``num_token_padding`` are left unwritten, as in the reference."""
    from .sgl_kernel import sgl_per_tensor_quant_fp8, sgl_per_token_quant_fp8

    assert input.ndim == 2, f"Expected 2D input tensor, got {input.ndim}D"
    shape = input.shape
    if num_token_padding:
        shape = (max(num_token_padding, input.shape[0]), shape[1])
    output = torch.empty(shape, device=input.device, dtype=fp8_dtype)
    if scale is None:
        if use_per_token_if_dynamic:
            scale = torch.empty((shape[0], 1), device=input.device, dtype=torch.float32)
            sgl_per_token_quant_fp8(input, output[: input.shape[0]], scale[: input.shape[0]])
        else:
            scale = torch.zeros(1, device=input.device, dtype=torch.float32)
            sgl_per_tensor_quant_fp8(input, output, scale, is_static=False)
    else:
        assert scale.numel() == 1, f"Expected scalar scale, got numel={scale.numel()}"
        sgl_per_tensor_quant_fp8(input, output, scale, is_static=True)
    return output, scale


def sglang_per_token_group_quant_int8(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    dtype: torch.dtype = torch.int8,
    enable_v2: Optional[bool] = None,
):
    """python/sglang/srt/layers/quantization/int8_kernel.py:183-218: row-major fp32 scales, int8 codes."""
    assert x.shape[-1] % group_size == 0, "the last dimension of `x` cannot be divisible by `group_size`"
    assert x.is_contiguous(), "`x` is not contiguous"
    iinfo = torch.iinfo(dtype)
    x_q = torch.empty_like(x, device=x.device, dtype=dtype)
    x_s = torch.empty(x.shape[:-1] + (x.shape[-1] // group_size,), device=x.device, dtype=torch.float32)
    if x.numel() > 0:
        sgl_per_token_group_quant_8bit(
            x, x_q, x_s, group_size, eps, float(iinfo.min), float(iinfo.max), enable_v2=enable_v2
        )
    return x_q, x_s


def sglang_per_token_group_quant_8bit(
    x: torch.Tensor,
    group_size: int,
    dst_dtype: torch.dtype,
    eps: float = 1e-10,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    scale_ue8m0: bool = False,
    fuse_silu_and_mul: bool = False,
    masked_m: Optional[torch.Tensor] = None,
    enable_v2: Optional[bool] = None,
):
    """fp8_kernel.py:531-570."""
    if dst_dtype == torch.int8:
        assert not column_major_scales
        assert not scale_tma_aligned
        assert not fuse_silu_and_mul
        assert masked_m is None
        return sglang_per_token_group_quant_int8(x=x, group_size=group_size, eps=eps, dtype=dst_dtype, enable_v2=enable_v2)

    return sglang_per_token_group_quant_fp8(
        x=x,
        group_size=group_size,
        eps=eps,
        column_major_scales=column_major_scales,
        scale_tma_aligned=scale_tma_aligned,
        scale_ue8m0=scale_ue8m0,
        fuse_silu_and_mul=fuse_silu_and_mul,
        masked_m=masked_m,
        enable_v2=enable_v2,
    )


def prepare_block_fp8_matmul_inputs(
    A: torch.Tensor,
    B: torch.Tensor,
    As: torch.Tensor,
    Bs: torch.Tensor,
    block_size: List[int],
    output_dtype: torch.dtype = torch.float16,
):
    """Shape contract of fp8_kernel.py:999-1044: fp32 scales, or int32 words holding four UE8M0 exponent bytes along K
    (``As`` [..., ceil(ceil(K/bk)/4)], ``Bs`` [N, ceil(ceil(K/bk)/4)], one row of words per weight row)."""
    assert len(block_size) == 2
    block_n, block_k = block_size[0], block_size[1]

    assert A.shape[-1] == B.shape[-1]
    assert A.shape[:-1] == As.shape[:-1]
    assert A.is_contiguous()

    if As.dtype == torch.float:
        assert ceil_div(A.shape[-1], block_k) == As.shape[-1]
    elif As.dtype == torch.int:
        assert ceil_div(ceil_div(A.shape[-1], block_k), 4) == As.shape[-1], f"{A.shape=} {As.shape=} {block_size=}"
    else:
        raise NotImplementedError

    M = A.numel() // A.shape[-1]

    assert B.ndim == 2
    assert B.is_contiguous()
    assert Bs.ndim == 2
    N, K = B.shape

    if Bs.dtype == torch.float:
        assert ceil_div(N, block_n) == Bs.shape[0]
        assert ceil_div(K, block_k) == Bs.shape[1]
    elif Bs.dtype == torch.int:
        assert N == Bs.shape[0], f"{B.shape=} {Bs.shape=} {block_size=}"
        assert ceil_div(ceil_div(K, block_k), 4) == Bs.shape[1], f"{B.shape=} {Bs.shape=} {block_size=}"
    else:
        raise NotImplementedError

    C_shape = A.shape[:-1] + (N,)
    C = A.new_empty(C_shape, dtype=output_dtype)

    return M, N, K, C


def _unpack_ue8m0_words(words: torch.Tensor, groups: int) -> torch.Tensor:
    """int32 words [..., ceil(groups/4)] with exponent byte j of word w belonging to K group 4 w + j -> fp32 powers of two
    [..., groups] (the inverse of the packing of per_token_group_quant_8bit_v2.cu:84-90, :305-329)."""
    bytes_ = torch.stack([(words >> (8 * j)) & 0xFF for j in range(4)], dim=-1).reshape(*words.shape[:-1], -1)[..., :groups]
    return (bytes_.to(torch.int32) << 23).view(torch.float32)


def w8a8_block_fp8_matmul(
    A: torch.Tensor,
    B: torch.Tensor,
    As: torch.Tensor,
    Bs: torch.Tensor,
    block_size: List[int],
    output_dtype: torch.dtype = torch.float16,
) -> torch.Tensor:
    """Block-wise quantized matmul, fp8_kernel.py:1068-1164.  ``B`` is the weight ``[N, K]`` as
    stored, ``Bs`` its ``[ceil(N/128), ceil(K/128)]`` scales, ``As`` the per-token-group scales of
    ``A``; N and K may be ragged with respect to the 128x128 blocks.  Scales packed as UE8M0 exponent bytes in int32
    words (the DeepGEMM operand format, :1016-1019, :1034-1039) are taken as they are when both operands carry them - the
    matrix instruction applies the exponents - and are expanded to fp32 first when only one side is packed."""
    M, N, K, C = prepare_block_fp8_matmul_inputs(A, B, As, Bs, block_size, output_dtype)
    if list(block_size) != [128, 128]:
        raise NotImplementedError("only 128x128 weight blocks with 1x128 activation groups are built")
    assert A.dtype == fp8_dtype and B.dtype == fp8_dtype
    assert output_dtype in (torch.float16, torch.bfloat16, torch.float32)
    if M == 0:
        return C
    As2d = As.reshape(M, As.shape[-1]) if As.dim() != 2 else As
    kb = ceil_div(K, 128)
    if As.dtype == torch.int32 and Bs.dtype == torch.int32 and output_dtype != torch.float32:
        if M > 1 and As2d.stride(0) != 1:
            # the kernels read a token's words with stride 1 along tokens (the layout the quantizer writes)
            As2d = As2d.t().contiguous().t()
        return ops.fp8_blockwise_mm_ue8m0(A.view(M, K), B, As2d, Bs, output_dtype).view(C.shape)
    if As.dtype == torch.int32:
        As2d = _unpack_ue8m0_words(As2d, kb)
    if Bs.dtype == torch.int32:
        Bs = _unpack_ue8m0_words(Bs[::128], kb)
    ops.block_fp8_matmul(A.view(M, K), B, As2d, Bs, C.view(M, N))
    return C


# The reference's callers import the kernel under this name (fp8_utils.py:281-301).
w8a8_block_fp8_matmul_triton = w8a8_block_fp8_matmul
