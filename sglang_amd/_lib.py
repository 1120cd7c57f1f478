"""Loader of ``libmi355_qlinear.so`` and typed ctypes prototypes of its C ABI.

There is no fallback: if the library is missing the import of any operator fails with a
clear message.  ``include/mi355_qlinear.h`` is the authoritative declaration; the prototypes
below mirror it one to one.
"""
from __future__ import annotations

import ctypes
import os

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_PATH = os.path.join(_CSRC, "libmi355_qlinear.so")
ABI_VERSION = 1

# enum values of include/mi355_qlinear.h
F32, F16, BF16, FP8_E4M3FN, I8, I32 = range(6)
QUANT_DIV, QUANT_RCP, QUANT_MUL = range(3)
SCALE_F32, SCALE_UE8M0_PACKED = range(2)
NOALLOC_SCRATCH_BYTES = 32 << 20

EXPORTS = (
    "mi355_qlinear_abi_version",
    "mi355_qlinear_init",
    "mi355_last_error",
    "mi355_group_quant_8bit",
    "mi355_fp8_blockwise_mm_workspace_bytes",
    "mi355_fp8_blockwise_mm",
    "mi355_fp8_blockwise_mm_noalloc",
    "mi355_fp8_blockwise_mm_kloop_ceiling",
    "mi355_probe_fp8_mfma_stream",
    "mi355_probe_int8_mfma_stream",
    "mi355_fp8_blockwise_mm_ue8m0_workspace_bytes",
    "mi355_fp8_blockwise_mm_ue8m0",
    "mi355_fp8_blockwise_scaled_grouped_mm_workspace_bytes",
    "mi355_fp8_blockwise_scaled_grouped_mm_plan",
    "mi355_fp8_blockwise_scaled_grouped_mm",
    "mi355_int8_scaled_mm_workspace_bytes",
    "mi355_int8_scaled_mm",
    "mi355_fp8_blockwise_mm_plan",
    "mi355_fp8_block_linear_plan",
    "mi355_int8_scaled_mm_plan",
    "mi355_route_constant_count",
    "mi355_route_constant_name",
    "mi355_route_constant_value",
    "mi355_gemm_plan_perturbed",
    "mi355_per_token_quant_int8",
    "mi355_per_token_quant_int8_sum",
    "mi355_per_token_quant_fp8",
    "mi355_row_group_quant_fp8",
    "mi355_per_tensor_quant_fp8",
    "mi355_silu_mul_group_quant_fp8",
    "mi355_block_cast_to_fp8",
    "mi355_block_dequant_fp8",
    "mi355_fp8_scaled_mm_workspace_bytes",
    "mi355_fp8_scaled_mm",
    "mi355_fp8_block_linear_workspace_bytes",
    "mi355_fp8_block_linear",
    "mi355_fp8_block_linear_mode",
    "mi355_int8_linear_workspace_bytes",
    "mi355_int8_linear",
    "mi355_fp8_per_token_linear_workspace_bytes",
    "mi355_fp8_per_token_linear",
    "mi355_fp8_block_linear_ue8m0_workspace_bytes",
    "mi355_fp8_block_linear_ue8m0",
)

_lib = None


class Mi355Error(RuntimeError):
    """A C-ABI call returned a non-zero status; the message is the library's own."""


def build() -> str:
    """Compile the library in-tree with the Makefile beside the sources (cross-compiles without a GPU)."""
    import subprocess

    subprocess.run(["make", "-C", _CSRC, "-B", "-j8", "libmi355_qlinear.so"], check=True)
    return LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C {_CSRC}` (or __graft_entry__.build()). "
            "The quantized-linear operators have no other implementation."
        )
    # The library links against libamdhip64; a process that also runs PyTorch must end up with ONE HIP runtime, the one
    # torch ships, so torch is loaded first (a library loaded before it would pull in the system copy as a second
    # runtime, which then sees no device).
    import torch  # noqa: F401

    L = ctypes.CDLL(LIB_PATH)
    i64, i32, f32, vp, sz = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t
    L.mi355_qlinear_abi_version.restype = i32
    L.mi355_last_error.restype = ctypes.c_char_p
    L.mi355_group_quant_8bit.argtypes = [vp, i32, vp, i32, vp, i64, i64, i32, f32, f32, f32, i32, i32, f32, i64, i64, vp]
    L.mi355_group_quant_8bit.restype = i32
    L.mi355_fp8_blockwise_mm_workspace_bytes.argtypes = [i64, i64, i64]
    L.mi355_fp8_blockwise_mm_workspace_bytes.restype = sz
    L.mi355_fp8_blockwise_mm.argtypes = [vp, vp, vp, vp, vp, i32] + [i64] * 10 + [vp, sz, vp]
    L.mi355_fp8_blockwise_mm.restype = i32
    L.mi355_fp8_blockwise_mm_ue8m0_workspace_bytes.argtypes = [i64, i64, i64]
    L.mi355_fp8_blockwise_mm_ue8m0_workspace_bytes.restype = sz
    L.mi355_fp8_blockwise_mm_ue8m0.argtypes = [vp, vp, vp, vp, vp, vp, i32] + [i64] * 9 + [vp, sz, vp]
    L.mi355_fp8_blockwise_mm_ue8m0.restype = i32
    L.mi355_fp8_blockwise_mm_noalloc.argtypes = [vp, vp, vp, vp, vp, i32] + [i64] * 10 + [vp]
    L.mi355_fp8_blockwise_mm_noalloc.restype = i32
    L.mi355_fp8_blockwise_mm_kloop_ceiling.argtypes = [vp, vp, vp, vp, vp, i32] + [i64] * 10 + [vp]
    L.mi355_fp8_blockwise_mm_kloop_ceiling.restype = i32
    L.mi355_probe_fp8_mfma_stream.argtypes = [i32, i32, i32, vp, vp, vp, vp]
    L.mi355_probe_fp8_mfma_stream.restype = i32
    L.mi355_probe_int8_mfma_stream.argtypes = [i32, i32, i32, vp, vp, vp, vp]
    L.mi355_probe_int8_mfma_stream.restype = i32
    L.mi355_fp8_blockwise_scaled_grouped_mm_workspace_bytes.argtypes = [i64, i64, i64, i64]
    L.mi355_fp8_blockwise_scaled_grouped_mm_workspace_bytes.restype = sz
    L.mi355_fp8_blockwise_scaled_grouped_mm_plan.argtypes = [i64, i64, i64, i64, ctypes.c_char_p, sz]
    L.mi355_fp8_blockwise_scaled_grouped_mm_plan.restype = i32
    L.mi355_fp8_blockwise_scaled_grouped_mm.argtypes = [vp, vp, vp, vp, vp, i32, vp, vp] + [i64] * 13 + [vp, sz, vp]
    L.mi355_fp8_blockwise_scaled_grouped_mm.restype = i32
    L.mi355_int8_scaled_mm_workspace_bytes.argtypes = [i64, i64, i64]
    L.mi355_int8_scaled_mm_workspace_bytes.restype = sz
    L.mi355_int8_scaled_mm.argtypes = [vp, vp, vp, vp, vp, vp, i32] + [i64] * 6 + [vp, sz, vp]
    L.mi355_int8_scaled_mm.restype = i32
    for fn in (L.mi355_fp8_blockwise_mm_plan, L.mi355_int8_scaled_mm_plan):
        fn.argtypes = [i64, i64, i64, i32, ctypes.c_char_p, sz]
        fn.restype = i32
    L.mi355_fp8_block_linear_plan.argtypes = [i64, i64, i64, ctypes.c_char_p, sz]
    L.mi355_fp8_block_linear_plan.restype = i32
    L.mi355_per_token_quant_int8.argtypes = [vp, i32, vp, vp, i64, i64, vp]
    L.mi355_per_token_quant_int8.restype = i32
    L.mi355_per_token_quant_int8_sum.argtypes = [vp, i32, vp, vp, vp, i64, i64, vp]
    L.mi355_per_token_quant_int8_sum.restype = i32
    L.mi355_per_token_quant_fp8.argtypes = [vp, i32, vp, vp, i64, i64, vp]
    L.mi355_per_token_quant_fp8.restype = i32
    L.mi355_row_group_quant_fp8.argtypes = [vp, i32, vp, vp, i64, i64, ctypes.c_float, i32, vp]
    L.mi355_row_group_quant_fp8.restype = i32
    L.mi355_per_tensor_quant_fp8.argtypes = [vp, i32, vp, vp, i64, i32, vp, i64, vp]
    L.mi355_per_tensor_quant_fp8.restype = i32
    L.mi355_silu_mul_group_quant_fp8.argtypes = [vp, i32, vp, vp, i64, i64, i64, vp, i64, i64, vp]
    L.mi355_silu_mul_group_quant_fp8.restype = i32
    L.mi355_block_cast_to_fp8.argtypes = [vp, i32, vp, vp, i64, i64, vp]
    L.mi355_block_cast_to_fp8.restype = i32
    L.mi355_block_dequant_fp8.argtypes = [vp, vp, vp, i32, i64, i64, vp]
    L.mi355_block_dequant_fp8.restype = i32
    L.mi355_fp8_scaled_mm_workspace_bytes.argtypes = [i64, i64, i64]
    L.mi355_fp8_scaled_mm_workspace_bytes.restype = sz
    L.mi355_fp8_scaled_mm.argtypes = [vp, vp, vp, vp, vp, vp, i32] + [i64] * 6 + [vp, sz, vp]
    L.mi355_fp8_scaled_mm.restype = i32
    L.mi355_fp8_block_linear_workspace_bytes.argtypes = [i64, i64, i64]
    L.mi355_fp8_block_linear_workspace_bytes.restype = sz
    L.mi355_fp8_block_linear.argtypes = [vp, i32, vp, vp, i64, i64, vp, vp, i32] + [i64] * 5 + [vp, sz, vp]
    L.mi355_fp8_block_linear.restype = i32
    L.mi355_fp8_block_linear_mode.argtypes = [vp, i32, i32, vp, vp, i64, i64, vp, vp, i32] + [i64] * 5 + [vp, sz, vp]
    L.mi355_fp8_block_linear_mode.restype = i32
    L.mi355_int8_linear_workspace_bytes.argtypes = [i64, i64, i64]
    L.mi355_int8_linear_workspace_bytes.restype = sz
    L.mi355_int8_linear.argtypes = [vp, i32, vp, vp, vp, vp, i32] + [i64] * 5 + [vp, sz, vp]
    L.mi355_int8_linear.restype = i32
    L.mi355_fp8_per_token_linear_workspace_bytes.argtypes = [i64, i64, i64]
    L.mi355_fp8_per_token_linear_workspace_bytes.restype = sz
    L.mi355_fp8_per_token_linear.argtypes = [vp, i32, vp, vp, vp, vp, i32] + [i64] * 5 + [vp, sz, vp]
    L.mi355_fp8_per_token_linear.restype = i32
    L.mi355_fp8_block_linear_ue8m0_workspace_bytes.argtypes = [i64, i64, i64]
    L.mi355_fp8_block_linear_ue8m0_workspace_bytes.restype = sz
    L.mi355_fp8_block_linear_ue8m0.argtypes = [vp, i32, vp, vp, i64, i64, vp, vp, i32] + [i64] * 5 + [vp, sz, vp]
    L.mi355_fp8_block_linear_ue8m0.restype = i32
    L.mi355_route_constant_count.restype = i32
    L.mi355_route_constant_name.argtypes = [i32]
    L.mi355_route_constant_name.restype = ctypes.c_char_p
    L.mi355_route_constant_value.argtypes = [i32]
    L.mi355_route_constant_value.restype = ctypes.c_double
    L.mi355_gemm_plan_perturbed.argtypes = [i32, i64, i64, i64, i32, i32, ctypes.c_double, ctypes.c_char_p, sz]
    L.mi355_gemm_plan_perturbed.restype = i32
    got = L.mi355_qlinear_abi_version()
    if got != ABI_VERSION:
        raise ImportError(f"{LIB_PATH} has ABI version {got}, this package needs {ABI_VERSION}: rebuild it")
    _lib = L
    return L


def gemm_plan(kind: str, M: int, N: int, K: int, aligned: bool = True) -> dict:
    """Kernel and tiling the library would use for an FP8 (`kind` "fp8") or INT8 ("int8") GEMM of this shape:
    {"kernel": str, "bm": int, "bn": int, "splits": int, "kb_per_split": int, "groups_per_wg": int, "aligned": int, "stages": int}."""
    fn = {"fp8": lib().mi355_fp8_blockwise_mm_plan, "int8": lib().mi355_int8_scaled_mm_plan}[kind]
    buf = ctypes.create_string_buffer(256)
    check(fn(M, N, K, int(aligned), buf, len(buf)))
    out = {}
    for item in buf.value.decode().split():
        k, v = item.split("=")
        out[k] = v if k == "kernel" else int(v)
    return out


def block_linear_plan(M: int, N: int, K: int) -> dict:
    """Plan of the one-call block-FP8 linear: `gemm_plan`'s keys plus "quantizer": "fused" (the GEMM kernel quantizes the
    tokens in its prologue) or "launch" (a quantizer launch in front of the GEMM)."""
    buf = ctypes.create_string_buffer(256)
    check(lib().mi355_fp8_block_linear_plan(M, N, K, buf, len(buf)))
    out = {}
    for item in buf.value.decode().split():
        k, v = item.split("=")
        out[k] = v if k in ("kernel", "quantizer") else int(v)
    return out


def route_constants() -> dict:
    """The dispatcher's measured time-model constants, name -> value, in table order."""
    L = lib()
    return {L.mi355_route_constant_name(i).decode(): L.mi355_route_constant_value(i) for i in range(L.mi355_route_constant_count())}


def gemm_plan_perturbed(kind: str, M: int, N: int, K: int, constant: int, factor: float, aligned: bool = True) -> dict:
    """`gemm_plan` with the `constant`-th entry of the dispatcher's constants table multiplied by `factor`."""
    buf = ctypes.create_string_buffer(256)
    check(lib().mi355_gemm_plan_perturbed(int(kind == "fp8"), M, N, K, int(aligned), constant, factor, buf, len(buf)))
    out = {}
    for item in buf.value.decode().split():
        k, v = item.split("=")
        out[k] = v if k == "kernel" else int(v)
    return out


def grouped_gemm_plan(num_experts: int, total_m: int, N: int, K: int) -> dict:
    """Tiling of the grouped FP8 GEMM for this many experts and stacked rows: {"kernel": str, "small_tile": "64x256" |
    "128x256", "max_big_tiles": int, "max_small_tiles": int, "tiles_n": int}."""
    buf = ctypes.create_string_buffer(256)
    check(lib().mi355_fp8_blockwise_scaled_grouped_mm_plan(num_experts, total_m, N, K, buf, len(buf)))
    out = {}
    for item in buf.value.decode().split():
        k, v = item.split("=")
        out[k] = v if k in ("kernel", "small_tile") else int(v)
    return out


def check(status: int) -> None:
    """Raise the library's message as RuntimeError (NotImplementedError for unsupported cases)."""
    if status == 0:
        return
    msg = lib().mi355_last_error().decode("utf-8", "replace")
    if status == 2:
        raise NotImplementedError(msg)
    raise Mi355Error(msg)
