"""PyTorch-ROCm custom operators ``torch.ops.sgl_kernel.*`` backed by the gfx950 C ABI.

The operator names and schema strings are the reference's own
(sgl-kernel/csrc/common_extension.cc:158-181); the implementations are registered for the
``CUDA`` dispatch key, which is the HIP device under PyTorch-ROCm.  Each implementation
checks its arguments the way the reference's host function does (same conditions, same
wording, RuntimeError), allocates outputs and workspaces through torch's caching allocator
(so nothing here breaks HIP graph capture) and passes raw device pointers plus the current
stream to ``libmi355_qlinear.so``.
"""
from __future__ import annotations

import functools
from typing import Optional

import torch

from . import _lib
from ._lib import check, lib

_DT = {
    torch.float32: _lib.F32,
    torch.float16: _lib.F16,
    torch.bfloat16: _lib.BF16,
    torch.float8_e4m3fn: _lib.FP8_E4M3FN,
    torch.int8: _lib.I8,
    torch.int32: _lib.I32,
}

SCHEMAS = {
    "int8_scaled_mm": "int8_scaled_mm(Tensor mat_a, Tensor mat_b, Tensor scales_a, Tensor scales_b, "
    "ScalarType out_dtype, Tensor? bias) -> Tensor",
    "fp8_blockwise_scaled_mm": "fp8_blockwise_scaled_mm(Tensor mat_a, Tensor mat_b, Tensor scales_a, "
    "Tensor scales_b, ScalarType out_dtype) -> Tensor",
    "sgl_per_token_group_quant_8bit": "sgl_per_token_group_quant_8bit(Tensor input, Tensor output_q, "
    "Tensor output_s, int group_size, float eps, float fp8_min, float fp8_max, bool scale_ue8m0) -> ()",
    "sgl_per_token_group_quant_8bit_v2": "sgl_per_token_group_quant_8bit_v2(Tensor input, Tensor output_q, "
    "Tensor output_s, int group_size, float eps, float fp8_min, float fp8_max, bool scale_ue8m0, "
    "bool fuse_silu_and_mul, Tensor? masked_m) -> ()",
    "fp8_scaled_mm": "fp8_scaled_mm(Tensor mat_a, Tensor mat_b, Tensor scales_a, Tensor scales_b, ScalarType out_dtype, "
    "Tensor? bias) -> Tensor",
    "sgl_per_token_quant_fp8": "sgl_per_token_quant_fp8(Tensor input, Tensor output_q, Tensor output_s) -> ()",
    "sgl_per_tensor_quant_fp8": "sgl_per_tensor_quant_fp8(Tensor input, Tensor output_q, Tensor output_s, bool is_static) -> ()",
    "fp8_blockwise_scaled_grouped_mm": "fp8_blockwise_scaled_grouped_mm(Tensor output, Tensor a_ptrs, Tensor b_ptrs, "
    "Tensor out_ptrs, Tensor a_scales_ptrs, Tensor b_scales_ptrs, Tensor a, Tensor b, Tensor scales_a, Tensor scales_b, "
    "Tensor stride_a, Tensor stride_b, Tensor stride_c, Tensor layout_sfa, Tensor layout_sfb, Tensor problem_sizes, "
    "Tensor expert_offsets, Tensor workspace) -> ()",
    "es_fp8_blockwise_scaled_grouped_mm": "es_fp8_blockwise_scaled_grouped_mm(Tensor output, Tensor a, Tensor b, Tensor scales_a, "
    "Tensor scales_b, Tensor stride_a, Tensor stride_b, Tensor stride_d, Tensor problem_sizes, Tensor expert_offsets, "
    "Tensor workspace) -> ()",
}


_ready_devices = set()


def _stream() -> int:
    """The current HIP stream; on a device's first use, the library's per-device set-up (it must not fall inside a graph
    capture, which the first launch of a process otherwise might)."""
    dev = torch.cuda.current_device()
    if dev not in _ready_devices and not torch.cuda.is_current_stream_capturing():
        # (inside a capture the set-up is left alone: the two entry points that need it say so in their error)
        check(lib().mi355_qlinear_init())
        _ready_devices.add(dev)
    if _raw_stream is not None:  # the handle itself, without building a torch.cuda.Stream object around it (~3 us a call)
        return _raw_stream(dev)
    return torch.cuda.current_stream().cuda_stream


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


@functools.lru_cache(maxsize=8192)
def _workspace_bytes(query: str, *dims: int) -> int:
    """Workspace size of an entry point for a shape (the `<entry>_workspace_bytes` query): a pure function of the shape,
    asked once per shape."""
    return int(getattr(lib(), query)(*dims))


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _check_input(t: torch.Tensor, name: str) -> None:
    # CHECK_INPUT of sgl-kernel/include/utils.h:193-212
    _require(t.is_cuda, f"{name} must be a CUDA tensor")
    _require(t.is_contiguous(), f"{name} must be contiguous")


# ---------------------------------------------------------------- group quantizer

def _group_quant(input, output_q, output_s, group_size, eps, qmin, qmax, scale_ue8m0, mode, pow2_floor, op):
    _check_input(input, "input")
    _check_input(output_q, "output_q")
    _require(input.numel() % group_size == 0, f"CHECK_EQ(input.numel() % group_size, 0) failed in {op}")
    _require(output_s.dim() == 2, f"CHECK_EQ(output_s.dim(), 2) failed in {op}")
    _require(input.dtype in (torch.float32, torch.float16, torch.bfloat16), f"{op}: unsupported input dtype {input.dtype}")
    _require(output_q.dtype in (torch.float8_e4m3fn, torch.int8), f"{op}: unsupported output dtype {output_q.dtype}")
    _require(output_q.numel() == input.numel(), f"{op}: output_q must have as many elements as input")
    if input.numel() == 0:
        return
    K = input.size(-1)
    M = input.numel() // K
    _require(K % group_size == 0, f"{op}: the last dimension must be divisible by group_size")
    if (group_size == K and mode == _lib.QUANT_DIV and not scale_ue8m0 and output_q.dtype == torch.float8_e4m3fn
            and (group_size * input.element_size() > 2048 or group_size & (group_size - 1)) and output_s.dtype == torch.float32
            and (qmin, qmax) == (-448.0, 448.0)):
        # the whole row is one group (a weight quantized per output channel at load time): rows longer than the group
        # kernel's 2048 bytes, or not a power of two
        _require(output_s.numel() == M and output_s.is_contiguous(), f"{op}: output_s must hold one contiguous scale per row")
        check(lib().mi355_row_group_quant_fp8(input.data_ptr(), _DT[input.dtype], output_q.data_ptr(), output_s.data_ptr(),
                                              M, K, eps, _lib.QUANT_DIV, _stream()))
        return
    # same test as per_token_group_quant_8bit.cu:153 / per_token_group_quant_8bit_v2.cu:426
    column_major = output_s.stride(0) < output_s.stride(1)
    if scale_ue8m0:
        _require(column_major, f"{op}: scale_ue8m0 needs column-major scales")
        _require(output_s.dtype == torch.int32, f"{op}: packed UE8M0 scales are stored in an int32 tensor")
        kind, s_row, s_col = _lib.SCALE_UE8M0_PACKED, 1, output_s.stride(1)
    else:
        _require(output_s.dtype == torch.float32, f"{op}: output_s must be float32")
        kind = _lib.SCALE_F32
        # row-major scales are addressed by the flat group index, as in the reference kernels
        s_row, s_col = (1, output_s.stride(1)) if column_major else (K // group_size, 1)
    check(
        lib().mi355_group_quant_8bit(
            input.data_ptr(), _DT[input.dtype], output_q.data_ptr(), _DT[output_q.dtype], output_s.data_ptr(),
            M, K, group_size, eps, qmin, qmax, mode, kind, pow2_floor, s_row, s_col, _stream(),
        )
    )


def sgl_per_token_group_quant_8bit(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0):
    """sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:116-217: q = x / (amax / max)."""
    _group_quant(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0,
                 _lib.QUANT_DIV, 1e-10, "sgl_per_token_group_quant_8bit")


def _silu_mul_group_quant(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0, masked_m, op):
    """The fuse_silu_and_mul branch of per_token_group_quant_8bit_v2.cu:394-514: input [T, 2H] or, with masked_m,
    [E, T, 2H]; the reference instantiates it for column-major packed UE8M0 scales only (:455-470)."""
    if not (scale_ue8m0 and output_s.dtype == torch.int32 and output_s.dim() >= 2 and output_s.stride(-2) == 1 and group_size == 128
            and output_q.dtype == torch.float8_e4m3fn):
        raise NotImplementedError(f"{op}: fuse_silu_and_mul is built for group 128, e4m3fn codes and column-major packed "
                                  "UE8M0 scales, the one combination the reference instantiates")
    _check_input(input, "input")
    _check_input(output_q, "output_q")
    _require(input.numel() > 0, f"{op}: input.numel() > 0")
    _require(abs(1e-10 - eps) < 1e-13, f"{op}: eps must be 1e-10")
    masked = masked_m is not None
    _require(output_s.dim() == (3 if masked else 2), f"{op}: output_s.dim() == {3 if masked else 2}")
    _require(input.dim() == output_s.dim(), f"{op}: input and output_s ranks differ")
    _require(input.dtype in (torch.float16, torch.bfloat16), f"{op}: input must be float16 or bfloat16")
    _require((fp8_min, fp8_max) == (-448.0, 448.0), f"{op}: CHECK_EQ(dst_dtype_info::MIN/MAX, min_8bit/max_8bit) failed")
    H = output_q.size(-1)
    T = output_q.size(-2)
    E = input.size(0) if masked else 1
    _require(input.size(-1) == 2 * H and input.size(-2) == T, f"{op}: input must be [..., tokens, 2 * hidden]")
    _require(H % 128 == 0, f"{op}: hidden size must be a multiple of 128")
    _require(output_s.size(-2) == T and output_s.size(-1) * 4 >= H // 128, f"{op}: output_s shape mismatch")
    mm = None
    if masked:
        _require(masked_m.is_cuda and masked_m.dtype == torch.int32 and masked_m.numel() == E and masked_m.is_contiguous(),
                 f"{op}: masked_m must be a contiguous int32 CUDA tensor with one entry per expert")
        mm = masked_m.data_ptr()
    check(lib().mi355_silu_mul_group_quant_fp8(input.data_ptr(), _DT[input.dtype], output_q.data_ptr(), output_s.data_ptr(),
                                               E, T, H, mm, output_s.stride(0) if masked else 0, output_s.stride(-1), _stream()))


def sgl_per_token_group_quant_8bit_v2(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0,
                                      fuse_silu_and_mul, masked_m):
    """sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:394-514: q = x * (max / amax)."""
    op = "sgl_per_token_group_quant_8bit_v2"
    if fuse_silu_and_mul:
        return _silu_mul_group_quant(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0, masked_m, op)
    if masked_m is not None:
        raise NotImplementedError(f"{op}: masked_m without fuse_silu_and_mul has no kernel in the reference either")
    _require(input.numel() > 0, f"{op}: input.numel() > 0")
    _require(abs(1e-10 - eps) < 1e-13, f"{op}: eps must be 1e-10")
    _require(group_size in (16, 32, 64, 128), "Unsupported group_size")
    _require(input.dtype in (torch.float16, torch.bfloat16), f"{op}: input must be float16 or bfloat16")
    want = (-448.0, 448.0) if output_q.dtype == torch.float8_e4m3fn else (-128.0, 127.0)
    _require((fp8_min, fp8_max) == want, f"{op}: CHECK_EQ(dst_dtype_info::MIN/MAX, min_8bit/max_8bit) failed")
    _group_quant(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0, _lib.QUANT_MUL, 0.0, op)


# ---------------------------------------------------------------- blockwise FP8 GEMM

def fp8_blockwise_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype):
    """sgl-kernel/csrc/gemm/fp8_blockwise_gemm_kernel.cu:368-465."""
    _require(mat_a.is_cuda, "mat_a must be a CUDA tensor")
    _require(mat_b.is_cuda, "mat_b must be a CUDA tensor")
    _require(mat_a.dim() == 2, "mat_a must be a 2D tensor")
    _require(mat_b.dim() == 2, "mat_b must be a 2D tensor")
    _require(mat_a.stride(1) == 1, "mat_a must be a row major tensor")
    _require(mat_b.stride(0) == 1, "mat_b must be a column major tensor")
    _require(mat_a.size(1) == mat_b.size(0), "mat_a and mat_b shapes cannot be multiplied")
    _require((mat_a.size(1) * mat_a.element_size()) % 16 == 0, "mat_a must be multiple of 16 bytes for memory alignment")
    _require((mat_b.size(0) * mat_b.element_size()) % 16 == 0, "mat_b must be multiple of 16 bytes for memory alignment")
    _require(mat_a.dtype == torch.float8_e4m3fn, "mat_a must be Float8_e4m3fn")
    _require(mat_b.dtype == torch.float8_e4m3fn, "mat_b must be Float8_e4m3fn")
    _require(out_dtype in (torch.float16, torch.bfloat16), "out_dtype must be Half or BFloat16")

    def is_contiguous_vector(t):
        return t.is_contiguous() and (t.dim() == 1 or (t.dim() == 2 and min(t.shape) == 1))

    M, K = mat_a.shape
    N = mat_b.size(1)
    _require(scales_a.dim() == 2 and scales_b.dim() == 2, "scales must be 2D tensors")
    _require(M == scales_a.size(0), "size of scales_a is not matched")
    _require(K // 128 == scales_a.size(1), "size of scales_a is not matched")
    _require(scales_a.stride(0) == 1 or is_contiguous_vector(scales_a), "scales_a must be M major")
    _require(K // 128 == scales_b.size(0), "size of scales_b is not matched")
    _require(N // 128 == scales_b.size(1), "size of scales_b is not matched")
    _require(scales_b.stride(0) == 1 or is_contiguous_vector(scales_b), "scales_b must be K major")
    _require(scales_a.dtype == torch.float32, "scales_a must be Float32")
    _require(scales_b.dtype == torch.float32, "scales_b must be Float32")
    _require((N * torch.empty((), dtype=out_dtype).element_size()) % 16 == 0,
             "out must be multiple of 16 bytes for memory alignment")
    # the integer divisions above accept ragged K or N but leave the tail without scales
    _require(K % 128 == 0 and N % 128 == 0, "fp8_blockwise_scaled_mm needs K and N to be multiples of 128")
    out = torch.empty((M, N), dtype=out_dtype, device=mat_a.device)
    if M == 0:
        return out
    _launch_fp8_mm(mat_a, mat_b.data_ptr(), mat_b.stride(1), scales_a, scales_b.data_ptr(),
                   scales_b.stride(1), scales_b.stride(0), out, M, N, K)
    return out


def _launch_fp8_mm(a, b_ptr, ldb, sa, sb_ptr, sb_sn, sb_sk, out, M, N, K):
    L = lib()
    ws_bytes = _workspace_bytes("mi355_fp8_blockwise_mm_workspace_bytes", int(M), int(N), int(K))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device) if ws_bytes else None
    check(
        L.mi355_fp8_blockwise_mm(
            a.data_ptr(), b_ptr, sa.data_ptr(), sb_ptr, out.data_ptr(), _DT[out.dtype], M, N, K,
            a.stride(0), ldb, sa.stride(0), sa.stride(1), sb_sn, sb_sk, out.stride(0),
            ws.data_ptr() if ws is not None else None, ws_bytes, _stream(),
        )
    )


def block_fp8_matmul(A2d, B, As2d, Bs, out2d):
    """The ``w8a8_block_fp8_matmul`` contract on flattened operands: B [N, K] row-major weight,
    Bs [ceil(N/128), ceil(K/128)], As2d [M, ceil(K/128)] any strides, ragged N and K allowed."""
    M, K = A2d.shape
    N = B.shape[0]
    if M == 0:
        return out2d
    _launch_fp8_mm(A2d, B.data_ptr(), B.stride(0), As2d, Bs.data_ptr(), Bs.stride(0), Bs.stride(1), out2d, M, N, K)
    return out2d


def _workspace(nbytes: int, device) -> Optional[torch.Tensor]:
    return torch.empty(nbytes, dtype=torch.uint8, device=device) if nbytes else None


# ---------------------------------------------------------------- per-token x per-channel FP8 linear

def sgl_per_token_quant_fp8(input, output_q, output_s):
    """sgl-kernel/csrc/gemm/per_token_quant_fp8.cu:162-227."""
    _check_input(input, "input")
    _check_input(output_q, "output_q")
    _check_input(output_s, "output_s")
    _require(input.dim() == 2, "sgl_per_token_quant_fp8: input must be 2-D")
    M, K = input.shape
    _require(K % 8 == 0, f"Hidden dimension must be divisible by 8, but got {K}")
    _require(input.dtype in (torch.float32, torch.float16, torch.bfloat16), "sgl_per_token_quant_fp8: unsupported input dtype")
    _require(output_q.dtype == torch.float8_e4m3fn and output_q.numel() == input.numel(), "sgl_per_token_quant_fp8: output_q mismatch")
    _require(output_s.dtype == torch.float32 and output_s.numel() == M, "sgl_per_token_quant_fp8: output_s mismatch")
    if M:
        check(lib().mi355_per_token_quant_fp8(input.data_ptr(), _DT[input.dtype], output_q.data_ptr(), output_s.data_ptr(),
                                              M, K, _stream()))


def block_cast_to_fp8(x: torch.Tensor):
    """x [m, n] -> (e4m3fn [m, n], fp32 power-of-two scales [ceil(m/128), ceil(n/128)]): per_block_cast_to_fp8 of
    python/sglang/srt/layers/quantization/fp8_utils.py:487-500 as one kernel."""
    _require(x.is_cuda and x.dim() == 2, "block_cast_to_fp8: a 2-D CUDA tensor is expected")
    _require(x.dtype in (torch.float32, torch.float16, torch.bfloat16), "block_cast_to_fp8: unsupported dtype")
    x = x.contiguous()
    m, n = x.shape
    q = torch.empty((m, n), dtype=torch.float8_e4m3fn, device=x.device)
    s = torch.empty(((m + 127) // 128, (n + 127) // 128), dtype=torch.float32, device=x.device)
    check(lib().mi355_block_cast_to_fp8(x.data_ptr(), _DT[x.dtype], q.data_ptr(), s.data_ptr(), m, n, _stream()))
    return q, s


def block_dequant_fp8(q: torch.Tensor, s: torch.Tensor, dtype: torch.dtype):
    """q [n, k] e4m3fn, s [ceil(n/128), ceil(k/128)] -> [n, k] of `dtype`: block_quant_dequant (fp8_utils.py:392-413)."""
    _require(q.is_cuda and q.dim() == 2 and q.dtype == torch.float8_e4m3fn, "block_dequant_fp8: a 2-D e4m3fn CUDA tensor is expected")
    n, k = q.shape
    _require(tuple(s.shape) == ((n + 127) // 128, (k + 127) // 128), "block_dequant_fp8: scale shape mismatch")
    _require(dtype in (torch.float32, torch.float16, torch.bfloat16), "block_dequant_fp8: unsupported dtype")
    q = q.contiguous()
    s = s.to(torch.float32).contiguous()
    out = torch.empty((n, k), dtype=dtype, device=q.device)
    check(lib().mi355_block_dequant_fp8(q.data_ptr(), s.data_ptr(), out.data_ptr(), _DT[dtype], n, k, _stream()))
    return out


def sgl_per_tensor_quant_fp8(input, output_q, output_s, is_static):
    """sgl-kernel/csrc/gemm/per_tensor_quant_fp8.cu:102-130.  Dynamic mode merges block maxima into `output_s` with an
    atomic max, so the caller passes zeros (the reference's scaled_fp8_quant does)."""
    _check_input(input, "input")
    _check_input(output_q, "output_q")
    _check_input(output_s, "output_s")
    _require(input.dtype in (torch.float32, torch.float16, torch.bfloat16), "sgl_per_tensor_quant_fp8: unsupported input dtype")
    _require(output_q.dtype == torch.float8_e4m3fn and output_q.numel() >= input.numel(), "sgl_per_tensor_quant_fp8: output_q mismatch")
    _require(output_s.dtype == torch.float32 and output_s.numel() >= 1, "sgl_per_tensor_quant_fp8: output_s mismatch")
    check(lib().mi355_per_tensor_quant_fp8(input.data_ptr(), _DT[input.dtype], output_q.data_ptr(), output_s.data_ptr(),
                                           input.numel(), int(bool(is_static)), None, 0, _stream()))


def static_quant_fp8_repeat(input, output_q, scale, scale_rows):
    """Static per-tensor quantization that also writes the scale once per row (static_quant_fp8 with repeat_scale,
    python/sglang/srt/layers/quantization/fp8_kernel.py:635-665)."""
    _check_input(input, "input")
    _check_input(output_q, "output_q")
    _require(scale.numel() == 1 and scale.dtype == torch.float32 and scale.is_cuda, "only supports per-tensor scale")
    _require(scale_rows.dtype == torch.float32 and scale_rows.is_contiguous(), "scale_rows must be contiguous float32")
    check(lib().mi355_per_tensor_quant_fp8(input.data_ptr(), _DT[input.dtype], output_q.data_ptr(), scale.data_ptr(),
                                           input.numel(), 1, scale_rows.data_ptr(), scale_rows.numel(), _stream()))


def fp8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias: Optional[torch.Tensor] = None):
    """sgl-kernel/csrc/gemm/fp8_gemm_kernel.cu:1450-1532."""
    _require(mat_a.is_cuda, "mat_a must be a CUDA tensor")
    _require(mat_b.is_cuda, "mat_b must be a CUDA tensor")
    _require(mat_a.dim() == 2, "mat_a must be a 2D tensor")
    _require(mat_b.dim() == 2, "mat_b must be a 2D tensor")
    _require(mat_a.stride(1) == 1, "mat_a must be a row major tensor")
    _require(mat_b.stride(0) == 1, "mat_b must be a column major tensor")
    _require(mat_a.size(1) == mat_b.size(0), "mat_a and mat_b shapes cannot be multiplied")
    _require((mat_a.size(1) * mat_a.element_size()) % 16 == 0, "mat_a must be multiple of 16 bytes for memory alignment")
    _require((mat_b.size(0) * mat_b.element_size()) % 16 == 0, "mat_b must be multiple of 16 bytes for memory alignment")
    _require(mat_a.dtype == torch.float8_e4m3fn, "mat_a must be Float8_e4m3fn")
    _require(mat_b.dtype == torch.float8_e4m3fn, "mat_b must be Float8_e4m3fn")
    _require(out_dtype in (torch.float16, torch.bfloat16), "out_dtype must be Half or BFloat16")
    M, K = mat_a.shape
    N = mat_b.size(1)
    _require(scales_a.numel() == M, "size of scales_a is not matched")
    _require(scales_b.numel() == N, "size of scales_b is not matched")
    _require(scales_a.is_contiguous(), "scales_a must be contiguous")
    _require(scales_b.is_contiguous(), "scales_b msut be contiguous")
    _require(scales_a.dtype == torch.float32, "scales_a must be Float32")
    _require(scales_b.dtype == torch.float32, "scales_b must be Float32")
    if bias is not None:
        _require(bias.numel() == N, "size of bias is not matched")
        _require(bias.is_contiguous(), "bias must be contiguous")
        _require(bias.dtype == out_dtype, "bias dtype must match output dtype")
    out = torch.empty((M, N), dtype=out_dtype, device=mat_a.device)
    _require((N * out.element_size()) % 16 == 0, "out must be multiple of 16 bytes for memory alignment")
    if M == 0:
        return out
    L = lib()
    ws_bytes = _workspace_bytes("mi355_fp8_scaled_mm_workspace_bytes", int(M), int(N), int(K))
    ws = _workspace(ws_bytes, mat_a.device)
    check(L.mi355_fp8_scaled_mm(mat_a.data_ptr(), mat_b.data_ptr(), scales_a.data_ptr(), scales_b.data_ptr(),
                                bias.data_ptr() if bias is not None else None, out.data_ptr(), _DT[out_dtype], M, N, K,
                                mat_a.stride(0), mat_b.stride(1), out.stride(0),
                                ws.data_ptr() if ws is not None else None, ws_bytes, _stream()))
    return out


def block_fp8_linear_ue8m0(x2d: torch.Tensor, weight: torch.Tensor, weight_words: torch.Tensor, bias: Optional[torch.Tensor],
                           out_dtype: torch.dtype) -> torch.Tensor:
    """One block-FP8 linear layer with packed power-of-two scales in one C-ABI call: x2d [M, K] (contiguous bf16/fp16,
    K % 128 == 0) is quantized per 1 x 128 group with UE8M0 scales into the workspace and multiplied with `weight` [N, K]
    e4m3fn, whose packed scale words are `weight_words` int32 [N, ceil(K/512)] (fp8_utils.transform_scale_ue8m0).  The
    result is that of the quantizer call of deepgemm_w8a8_block_fp8_linear_with_fallback followed by
    `fp8_blockwise_mm_ue8m0`, bit for bit."""
    _require(x2d.is_cuda and weight.is_cuda, "block_fp8_linear_ue8m0: operands must be CUDA tensors")
    _require(x2d.dim() == 2 and x2d.is_contiguous() and x2d.dtype in (torch.bfloat16, torch.float16),
             "block_fp8_linear_ue8m0: x must be a contiguous 2-D bf16/fp16 tensor")
    _require(weight.dim() == 2 and weight.stride(1) == 1 and weight.dtype == torch.float8_e4m3fn,
             "block_fp8_linear_ue8m0: weight must be a row-major Float8_e4m3fn matrix")
    M, K = x2d.shape
    N = weight.size(0)
    _require(weight.size(1) == K and K % 128 == 0, "block_fp8_linear_ue8m0: K must match and be a multiple of 128")
    kw = (K // 128 + 3) // 4
    _require(weight_words.dtype == torch.int32 and weight_words.dim() == 2 and weight_words.size(0) == N and weight_words.size(1) >= kw,
             f"block_fp8_linear_ue8m0: weight_words must be int32 [{N}, >= {kw}]")
    _require(out_dtype in (torch.float16, torch.bfloat16), "block_fp8_linear_ue8m0: out_dtype must be Half or BFloat16")
    if bias is not None:
        _require(bias.numel() == N and bias.is_contiguous() and bias.dtype == out_dtype,
                 "block_fp8_linear_ue8m0: bias must be a contiguous [N] tensor of the output dtype")
    out = torch.empty((M, N), dtype=out_dtype, device=x2d.device)
    if M == 0 or N == 0:
        return out
    L = lib()
    ws_bytes = _workspace_bytes("mi355_fp8_block_linear_ue8m0_workspace_bytes", int(M), int(N), int(K))
    ws = _workspace(ws_bytes, x2d.device)
    check(L.mi355_fp8_block_linear_ue8m0(x2d.data_ptr(), _DT[x2d.dtype], weight.data_ptr(), weight_words.data_ptr(),
                                         weight_words.stride(0), weight_words.stride(1),
                                         bias.data_ptr() if bias is not None else None, out.data_ptr(), _DT[out_dtype],
                                         M, N, K, weight.stride(0), out.stride(0), ws.data_ptr(), ws_bytes, _stream()))
    return out


def fp8_per_token_linear(x2d: torch.Tensor, weight_kn: torch.Tensor, weight_scale: torch.Tensor, bias: Optional[torch.Tensor],
                         out_dtype: torch.dtype) -> torch.Tensor:
    """One per-token x per-channel FP8 linear layer in one C-ABI call: per-token quantization of x2d [M, K] (contiguous
    bf16/fp16/fp32) into the workspace, then the GEMM with `weight_kn` [K, N] e4m3fn column-major, per-channel `weight_scale`
    ([N] fp32) and bias in its epilogue.  The result is that of `sgl_per_token_quant_fp8` followed by `fp8_scaled_mm`, bit
    for bit."""
    _require(x2d.is_cuda and weight_kn.is_cuda, "fp8_per_token_linear: operands must be CUDA tensors")
    _require(x2d.dim() == 2 and x2d.is_contiguous(), "fp8_per_token_linear: x must be a contiguous 2-D tensor")
    _require(x2d.dtype in (torch.float32, torch.float16, torch.bfloat16), "fp8_per_token_linear: unsupported input dtype")
    _require(weight_kn.dim() == 2 and weight_kn.stride(0) == 1 and weight_kn.dtype == torch.float8_e4m3fn,
             "fp8_per_token_linear: weight must be a column-major Float8_e4m3fn matrix [K, N]")
    M, K = x2d.shape
    N = weight_kn.size(1)
    _require(weight_kn.size(0) == K, "fp8_per_token_linear: x and weight shapes cannot be multiplied")
    _require(K % 16 == 0, "fp8_per_token_linear: K must be multiple of 16 bytes for memory alignment")
    _require(weight_scale.numel() == N and weight_scale.is_contiguous() and weight_scale.dtype == torch.float32,
             "fp8_per_token_linear: weight_scale must be a contiguous Float32 tensor of N elements")
    _require(out_dtype in (torch.float16, torch.bfloat16), "fp8_per_token_linear: out_dtype must be Half or BFloat16")
    _require(N % 8 == 0, "fp8_per_token_linear: out must be multiple of 16 bytes for memory alignment")
    if bias is not None:
        _require(bias.numel() == N and bias.is_contiguous() and bias.dtype == out_dtype,
                 "fp8_per_token_linear: bias must be a contiguous [N] tensor of the output dtype")
    out = torch.empty((M, N), dtype=out_dtype, device=x2d.device)
    if M == 0:
        return out
    L = lib()
    ws_bytes = _workspace_bytes("mi355_fp8_per_token_linear_workspace_bytes", int(M), int(N), int(K))
    ws = _workspace(ws_bytes, x2d.device)
    check(L.mi355_fp8_per_token_linear(x2d.data_ptr(), _DT[x2d.dtype], weight_kn.data_ptr(), weight_scale.data_ptr(),
                                       bias.data_ptr() if bias is not None else None, out.data_ptr(), _DT[out_dtype], M, N, K,
                                       weight_kn.stride(1), out.stride(0), ws.data_ptr(), ws_bytes, _stream()))
    return out


def block_fp8_linear(x2d: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
                     bias: Optional[torch.Tensor], out_dtype: torch.dtype, by_reciprocal: bool = False) -> torch.Tensor:
    """One block-FP8 linear layer (1x128 activation groups, 128x128 weight blocks) in one C-ABI call: the activation is
    quantized into the workspace, multiplied, and the bias is added in the GEMM epilogue.  x2d [M, K] contiguous
    bf16/fp16/fp32 with K % 128 == 0, weight [N, K] e4m3fn, weight_scale [ceil(N/128), K/128] (any strides).
    by_reciprocal: the quantizer computes q = x * (1 / s) (the reference's row-major-scale path, fp8_kernel.py:156-158)
    instead of q = x / s (its M-major-scale path)."""
    _require(x2d.is_cuda and weight.is_cuda, "block_fp8_linear: operands must be CUDA tensors")
    _require(x2d.dim() == 2 and x2d.is_contiguous(), "block_fp8_linear: x must be a contiguous 2-D tensor")
    _require(weight.dim() == 2 and weight.stride(1) == 1 and weight.dtype == torch.float8_e4m3fn,
             "block_fp8_linear: weight must be a row-major Float8_e4m3fn matrix")
    M, K = x2d.shape
    N = weight.size(0)
    _require(weight.size(1) == K and K % 128 == 0, "block_fp8_linear: K must match and be a multiple of 128")
    _require(tuple(weight_scale.shape) == ((N + 127) // 128, K // 128) and weight_scale.dtype == torch.float32,
             "block_fp8_linear: weight_scale must be float32 [ceil(N/128), K/128]")
    _require(out_dtype in (torch.float16, torch.bfloat16), "block_fp8_linear: out_dtype must be Half or BFloat16")
    if bias is not None:
        _require(bias.numel() == N and bias.is_contiguous() and bias.dtype == out_dtype,
                 "block_fp8_linear: bias must be a contiguous [N] tensor of the output dtype")
    out = torch.empty((M, N), dtype=out_dtype, device=x2d.device)
    if M == 0:
        return out
    L = lib()
    ws_bytes = _workspace_bytes("mi355_fp8_block_linear_workspace_bytes", int(M), int(N), int(K))
    ws = _workspace(ws_bytes, x2d.device)
    check(L.mi355_fp8_block_linear_mode(x2d.data_ptr(), _DT[x2d.dtype], 1 if by_reciprocal else 0, weight.data_ptr(),
                                        weight_scale.data_ptr(), weight_scale.stride(0), weight_scale.stride(1),
                                        bias.data_ptr() if bias is not None else None, out.data_ptr(), _DT[out_dtype],
                                        M, N, K, weight.stride(0), out.stride(0), ws.data_ptr(), ws_bytes, _stream()))
    return out


def fp8_blockwise_mm_ue8m0(a: torch.Tensor, b: torch.Tensor, a_words: torch.Tensor, b_words: torch.Tensor,
                           out_dtype: torch.dtype, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Blockwise FP8 GEMM with packed power-of-two scales on both sides: a [M, K] e4m3fn, b [N, K] e4m3fn (the weight as
    stored), a_words int32 [M, ceil(K/512)] and b_words int32 [N, ceil(K/512)], both with stride 1 along their first
    dimension (the layouts of create_per_token_group_quant_fp8_output_scale(scale_ue8m0=True) and
    fp8_utils.transform_scale_ue8m0).  What deep_gemm's gemm_nt_f8f8bf16 computes for the reference
    (python/sglang/srt/layers/quantization/fp8_kernel.py:1047-1065)."""
    _require(a.is_cuda and b.is_cuda, "fp8_blockwise_mm_ue8m0: operands must be CUDA tensors")
    _require(a.dim() == 2 and b.dim() == 2 and a.stride(1) == 1 and b.stride(1) == 1, "fp8_blockwise_mm_ue8m0: row-major operands expected")
    _require(a.dtype == torch.float8_e4m3fn and b.dtype == torch.float8_e4m3fn, "fp8_blockwise_mm_ue8m0: operands must be Float8_e4m3fn")
    M, K = a.shape
    N = b.size(0)
    _require(b.size(1) == K, "fp8_blockwise_mm_ue8m0: shapes cannot be multiplied")
    kw = (((K + 127) // 128) + 3) // 4
    for t, rows, name in ((a_words, M, "a_words"), (b_words, N, "b_words")):
        _require(t.dtype == torch.int32 and t.dim() == 2 and t.size(0) == rows and t.size(1) >= kw,
                 f"fp8_blockwise_mm_ue8m0: {name} must be int32 [{rows}, >= {kw}]")
    _require(M <= 1 or a_words.stride(0) == 1, "fp8_blockwise_mm_ue8m0: a_words must be packed along tokens (stride(0) == 1)")
    _require(out_dtype in (torch.float16, torch.bfloat16), "fp8_blockwise_mm_ue8m0: out_dtype must be Half or BFloat16")
    if bias is not None:
        _require(bias.numel() == N and bias.is_contiguous() and bias.dtype == out_dtype,
                 "fp8_blockwise_mm_ue8m0: bias must be a contiguous [N] tensor of the output dtype")
    out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    if M == 0 or N == 0:
        return out
    L = lib()
    ws_bytes = _workspace_bytes("mi355_fp8_blockwise_mm_ue8m0_workspace_bytes", int(M), int(N), int(K))
    ws = _workspace(ws_bytes, a.device)
    check(L.mi355_fp8_blockwise_mm_ue8m0(
        a.data_ptr(), b.data_ptr(), a_words.data_ptr(), b_words.data_ptr(), bias.data_ptr() if bias is not None else None,
        out.data_ptr(), _DT[out_dtype], M, N, K, a.stride(0), b.stride(0), a_words.stride(1), b_words.stride(0), b_words.stride(1),
        out.stride(0), ws.data_ptr() if ws is not None else None, ws_bytes, _stream()))
    return out


# ---------------------------------------------------------------- grouped FP8 GEMM (mixture-of-experts)

def _grouped_mm(op, output, a, b, scales_a, scales_b, problem_sizes, expert_offsets, workspace):
    """Checks common to both grouped entry points (fp8_blockwise_moe_kernel.cu:668-677, es_fp8_blockwise.cu:46-55), the
    layout checks the kernels need, and the call."""
    _require(problem_sizes.dim() == 2, "problem_sizes must be 2D tensor")
    _require(problem_sizes.size(1) == 3, "problem_sizes must have shape (num_experts, 3)")
    _require(problem_sizes.size(0) == expert_offsets.size(0), "Number of experts in problem_sizes must match expert_offsets")
    _require(problem_sizes.dtype == torch.int32, "problem_sizes must be int32")
    _require(a.dtype == torch.float8_e4m3fn, "a must be kFloat8_e4m3fn")
    _require(b.dtype == torch.float8_e4m3fn, "b must be kFloat8_e4m3fn")
    _require(output.dtype in (torch.bfloat16, torch.float16), "output must be bfloat16 or half")
    _require(scales_a.dtype == torch.float32, "scales_a must be float32")
    _require(scales_b.dtype == torch.float32, "scales_b must be float32")
    _require(expert_offsets.dtype == torch.int32 and expert_offsets.dim() == 1, "expert_offsets must be a 1D int32 tensor")
    _require(output.dim() == 2, "output must be 2D tensor")
    _require(a.dim() == 2, "a must be 2D tensor")
    _require(b.dim() == 3, "b must be 3D tensor")
    _require(scales_a.dim() == 2, "scales_a must be 2D tensor")
    _require(scales_b.dim() == 3, "scales_b must be 3D tensor")
    _require(workspace.dim() == 1, "workspace must be 1D tensor")
    _require(a.is_cuda and b.is_cuda and output.is_cuda and problem_sizes.is_cuda and expert_offsets.is_cuda,
             f"{op}: tensors must be CUDA tensors")
    total_m, K = a.shape
    E, Kb, N = b.shape
    _require(Kb == K and output.size(0) == total_m and output.size(1) == N and problem_sizes.size(0) == E,
             f"{op}: shapes do not fit together")
    _require(a.stride(1) == 1 and output.stride(1) == 1, f"{op}: a and output must be row-major")
    _require(b.stride(1) == 1 or K == 1, f"{op}: b must be column-major per expert ([E, K, N] view of [E, N, K] storage)")
    kb, nb = (K + 127) // 128, (N + 127) // 128
    _require(tuple(scales_a.shape) == (total_m, kb), f"{op}: scales_a must be [{total_m}, {kb}]")
    _require(tuple(scales_b.shape) == (E, kb, nb), f"{op}: scales_b must be [{E}, {kb}, {nb}]")
    _require(expert_offsets.is_contiguous() and problem_sizes.is_contiguous(), f"{op}: problem_sizes and expert_offsets must be contiguous")
    if total_m == 0 or N == 0 or E == 0:
        return
    L = lib()
    need = _workspace_bytes("mi355_fp8_blockwise_scaled_grouped_mm_workspace_bytes", int(E), int(total_m), int(N), int(K))
    ws = workspace
    if not (ws.is_cuda and ws.is_contiguous() and ws.numel() * ws.element_size() >= need and ws.data_ptr() % 256 == 0):
        ws = _workspace(need, a.device)
    check(L.mi355_fp8_blockwise_scaled_grouped_mm(
        a.data_ptr(), b.data_ptr(), scales_a.data_ptr(), scales_b.data_ptr(), output.data_ptr(), _DT[output.dtype],
        problem_sizes.data_ptr(), expert_offsets.data_ptr(), E, total_m, N, K, a.stride(0), b.stride(2), b.stride(0),
        scales_a.stride(0), scales_a.stride(1), scales_b.stride(0), scales_b.stride(2), scales_b.stride(1), output.stride(0),
        ws.data_ptr(), ws.numel() * ws.element_size(), _stream()))


def fp8_blockwise_scaled_grouped_mm(output, a_ptrs, b_ptrs, out_ptrs, a_scales_ptrs, b_scales_ptrs, a, b, scales_a, scales_b,
                                    stride_a, stride_b, stride_c, layout_sfa, layout_sfb, problem_sizes, expert_offsets,
                                    workspace):
    """sgl-kernel/csrc/moe/fp8_blockwise_moe_kernel.cu:650-810 (checks :668-706).  ``a`` [total_m, K] e4m3fn row-major,
    ``b`` [E, K, N] e4m3fn column-major per expert (storage [E, N, K]), ``scales_a`` fp32 [total_m, K/128], ``scales_b``
    fp32 [E, K/128, N/128] (storage [E, N/128, K/128]), ``problem_sizes`` int32 [E, 3] and ``expert_offsets`` int32 [E] on
    the device, ``output`` [total_m, N] written in place.  The pointer, stride and scale-layout tensors are scratch of the
    reference's kernels: they are type-checked like there and not used.  ``workspace`` is used when it is large enough
    (the reference's callers pass hundreds of megabytes), otherwise a temporary one is allocated."""
    for t, name in ((stride_a, "stride_a"), (stride_b, "stride_b"), (stride_c, "stride_c")):
        _require(t.dtype == torch.int64 and t.dim() == 1, f"{name} must be a 1D int64 tensor")
    for t, name in ((layout_sfa, "layout_sfa"), (layout_sfb, "layout_sfb")):
        _require(t.dtype == torch.int32 and t.dim() == 2, f"{name} must be a 2D int32 tensor")
    for t, name in ((a_ptrs, "a_ptrs"), (b_ptrs, "b_ptrs"), (out_ptrs, "out_ptrs"), (a_scales_ptrs, "a_scales_ptrs"),
                    (b_scales_ptrs, "b_scales_ptrs")):
        _require(t.dim() == 1, f"{name} must be 1D tensor")
    _grouped_mm("fp8_blockwise_scaled_grouped_mm", output, a, b, scales_a, scales_b, problem_sizes, expert_offsets, workspace)


def es_fp8_blockwise_scaled_grouped_mm(output, a, b, scales_a, scales_b, stride_a, stride_b, stride_d, problem_sizes,
                                       expert_offsets, workspace):
    """sgl-kernel/csrc/expert_specialization/es_fp8_blockwise.cu:33-170: the same computation on the same layouts without
    the caller-provided scratch tensors.  The reference sorts experts into low / middle / high row counts and runs one
    tile configuration on each; here the device-built schedule does that per tile (256-row tiles and a small-tile rest)."""
    _grouped_mm("es_fp8_blockwise_scaled_grouped_mm", output, a, b, scales_a, scales_b, problem_sizes, expert_offsets, workspace)


# ---------------------------------------------------------------- INT8 GEMM

def int8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias: Optional[torch.Tensor] = None):
    """sgl-kernel/csrc/gemm/int8_gemm_kernel.cu:663-747."""
    _require(mat_a.is_cuda, "mat_a must be a CUDA tensor")
    _require(mat_b.is_cuda, "mat_b must be a CUDA tensor")
    _require(mat_a.dim() == 2, "mat_a must be a 2D tensor")
    _require(mat_b.dim() == 2, "mat_b must be a 2D tensor")
    _require(mat_a.stride(1) == 1, "mat_a must be a row major tensor")
    _require(mat_b.stride(0) == 1, "mat_b must be a column major tensor")
    _require(mat_a.size(1) == mat_b.size(0), "mat_a and mat_b shapes cannot be multiplied")
    _require(mat_a.size(1) % 16 == 0, "mat_a.size(1) must be multiple of 16 for memory alignment")
    _require(mat_b.size(0) % 16 == 0, "mat_b.size(0) must be multiple of 16 for memory alignment")
    _require(mat_b.size(1) % 8 == 0, "mat_b.size(1) must be multiple of 8 for memory alignment")
    _require(mat_a.dtype == torch.int8, "mat_a must be Int8")
    _require(mat_b.dtype == torch.int8, "mat_b must be Int8")
    _require(out_dtype in (torch.float16, torch.bfloat16), "out_dtype must be Half or BFloat16")
    M, K = mat_a.shape
    N = mat_b.size(1)
    _require(scales_a.numel() == M, "size of scales_a is not matched")
    _require(scales_b.numel() == N, "size of scales_b is not matched")
    _require(scales_a.is_contiguous(), "scales_a must be contiguous")
    _require(scales_b.is_contiguous(), "scales_b msut be contiguous")
    _require(scales_a.dtype == torch.float32, "scales_a must be Float32")
    _require(scales_b.dtype == torch.float32, "scales_b must be Float32")
    if bias is not None:
        _require(bias.numel() == N, "size of bias is not matched")
        _require(bias.is_contiguous(), "bias must be contiguous")
        _require(bias.dtype == out_dtype, "bias dtype must match output dtype")
    out = torch.empty((M, N), dtype=out_dtype, device=mat_a.device)
    if M == 0:
        return out
    _launch_int8_mm(mat_a, mat_b, scales_a, scales_b, bias, out)
    return out


def int8_linear(x2d: torch.Tensor, weight_kn: torch.Tensor, weight_scale: torch.Tensor, bias: Optional[torch.Tensor],
                out_dtype: torch.dtype) -> torch.Tensor:
    """One INT8 linear layer in one C-ABI call: per-token quantization of x2d [M, K] (contiguous bf16/fp16/fp32) into the
    workspace, then the INT8 GEMM with `weight_kn` [K, N] int8 column-major, per-channel `weight_scale` ([N] fp32) and bias in
    its epilogue.  The result is that of `per_token_quant_int8` followed by `int8_scaled_mm`, bit for bit."""
    _require(x2d.is_cuda and weight_kn.is_cuda, "int8_linear: operands must be CUDA tensors")
    _require(x2d.dim() == 2 and x2d.is_contiguous(), "int8_linear: x must be a contiguous 2-D tensor")
    _require(x2d.dtype in (torch.float32, torch.float16, torch.bfloat16), "int8_linear: unsupported input dtype")
    _require(weight_kn.dim() == 2 and weight_kn.stride(0) == 1 and weight_kn.dtype == torch.int8,
             "int8_linear: weight must be a column-major Int8 matrix [K, N]")
    M, K = x2d.shape
    N = weight_kn.size(1)
    _require(weight_kn.size(0) == K, "int8_linear: x and weight shapes cannot be multiplied")
    _require(K % 16 == 0, "int8_linear: K must be multiple of 16 for memory alignment")
    _require(N % 8 == 0, "int8_linear: N must be multiple of 8 for memory alignment")
    _require(weight_scale.numel() == N and weight_scale.is_contiguous() and weight_scale.dtype == torch.float32,
             "int8_linear: weight_scale must be a contiguous Float32 tensor of N elements")
    _require(out_dtype in (torch.float16, torch.bfloat16), "int8_linear: out_dtype must be Half or BFloat16")
    if bias is not None:
        _require(bias.numel() == N and bias.is_contiguous() and bias.dtype == out_dtype,
                 "int8_linear: bias must be a contiguous [N] tensor of the output dtype")
    out = torch.empty((M, N), dtype=out_dtype, device=x2d.device)
    if M == 0:
        return out
    L = lib()
    ws_bytes = _workspace_bytes("mi355_int8_linear_workspace_bytes", int(M), int(N), int(K))
    ws = _workspace(ws_bytes, x2d.device)
    check(L.mi355_int8_linear(x2d.data_ptr(), _DT[x2d.dtype], weight_kn.data_ptr(), weight_scale.data_ptr(),
                              bias.data_ptr() if bias is not None else None, out.data_ptr(), _DT[out_dtype], M, N, K,
                              weight_kn.stride(1), out.stride(0), ws.data_ptr(), ws_bytes, _stream()))
    return out


def _launch_int8_mm(mat_a, mat_b, scales_a, scales_b, bias, out):
    M, K = mat_a.shape
    N = mat_b.size(1)
    L = lib()
    ws_bytes = _workspace_bytes("mi355_int8_scaled_mm_workspace_bytes", int(M), int(N), int(K))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=mat_a.device) if ws_bytes else None
    check(
        L.mi355_int8_scaled_mm(
            mat_a.data_ptr(), mat_b.data_ptr(),
            scales_a.data_ptr() if scales_a is not None else None,
            scales_b.data_ptr() if scales_b is not None else None,
            bias.data_ptr() if bias is not None else None, out.data_ptr(), _DT[out.dtype], M, N, K,
            mat_a.stride(0), mat_b.stride(1), out.stride(0),
            ws.data_ptr() if ws is not None else None, ws_bytes, _stream(),
        )
    )


def int8_mm_raw_accumulators(mat_a: torch.Tensor, mat_b: torch.Tensor) -> torch.Tensor:
    """int32 accumulators of ``int8_scaled_mm`` before its epilogue (same kernel, epilogue skipped)."""
    out = torch.empty((mat_a.size(0), mat_b.size(1)), dtype=torch.int32, device=mat_a.device)
    if mat_a.size(0):
        _launch_int8_mm(mat_a, mat_b, None, None, None, out)
    return out


def per_token_quant_int8(x2d: torch.Tensor, q: torch.Tensor, s: torch.Tensor, x_sum: Optional[torch.Tensor] = None) -> None:
    """Codes and scales of the rows of `x2d`; with `x_sum` ([M], the input's type) also the row sums."""
    M, K = x2d.shape
    if not M:
        return
    if x_sum is None:
        check(lib().mi355_per_token_quant_int8(x2d.data_ptr(), _DT[x2d.dtype], q.data_ptr(), s.data_ptr(), M, K, _stream()))
    else:
        _require(x_sum.dtype == x2d.dtype and x_sum.numel() == M and x_sum.is_contiguous(), "x_sum must be [M] in the input's type")
        check(lib().mi355_per_token_quant_int8_sum(x2d.data_ptr(), _DT[x2d.dtype], q.data_ptr(), s.data_ptr(), x_sum.data_ptr(), M, K,
                                                   _stream()))


# ---------------------------------------------------------------- registration

_registered = False
_torch_lib = None


def register() -> None:
    """Define the ``sgl_kernel`` operators (unless an installed sgl_kernel already did) and attach
    the gfx950 implementations to the CUDA (= HIP) dispatch key.  Idempotent."""
    global _registered, _torch_lib
    if _registered:
        return
    lib()  # fail now, loudly, if the native library is missing
    _torch_lib = torch.library.Library("sgl_kernel", "FRAGMENT")
    impls = {
        "int8_scaled_mm": int8_scaled_mm,
        "fp8_blockwise_scaled_mm": fp8_blockwise_scaled_mm,
        "sgl_per_token_group_quant_8bit": sgl_per_token_group_quant_8bit,
        "sgl_per_token_group_quant_8bit_v2": sgl_per_token_group_quant_8bit_v2,
        "fp8_scaled_mm": fp8_scaled_mm,
        "sgl_per_token_quant_fp8": sgl_per_token_quant_fp8,
        "sgl_per_tensor_quant_fp8": sgl_per_tensor_quant_fp8,
        "fp8_blockwise_scaled_grouped_mm": fp8_blockwise_scaled_grouped_mm,
        "es_fp8_blockwise_scaled_grouped_mm": es_fp8_blockwise_scaled_grouped_mm,
    }
    for name, fn in impls.items():
        if not hasattr(torch.ops.sgl_kernel, name):
            _torch_lib.define(SCHEMAS[name])
        _torch_lib.impl(name, fn, "CUDA")

    def _fake_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None):
        return mat_a.new_empty((mat_a.size(0), mat_b.size(1)), dtype=out_dtype)

    torch.library.register_fake("sgl_kernel::int8_scaled_mm", _fake_mm, lib=_torch_lib)
    torch.library.register_fake("sgl_kernel::fp8_blockwise_scaled_mm", _fake_mm, lib=_torch_lib)
    torch.library.register_fake("sgl_kernel::fp8_scaled_mm", _fake_mm, lib=_torch_lib)
    torch.library.register_fake("sgl_kernel::sgl_per_token_quant_fp8", lambda *a: None, lib=_torch_lib)
    torch.library.register_fake("sgl_kernel::sgl_per_tensor_quant_fp8", lambda *a: None, lib=_torch_lib)
    torch.library.register_fake("sgl_kernel::fp8_blockwise_scaled_grouped_mm", lambda *a: None, lib=_torch_lib)
    torch.library.register_fake("sgl_kernel::es_fp8_blockwise_scaled_grouped_mm", lambda *a: None, lib=_torch_lib)
    torch.library.register_fake("sgl_kernel::sgl_per_token_group_quant_8bit", lambda *a: None, lib=_torch_lib)
    torch.library.register_fake("sgl_kernel::sgl_per_token_group_quant_8bit_v2", lambda *a: None, lib=_torch_lib)
    _registered = True
