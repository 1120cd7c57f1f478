"""CPU-side checks of the drop-in boundary: the shared library loads, exports every symbol the
header declares, validates arguments before touching the device, and the Python operator
layer carries the reference's names, schemas and error wording.  No kernel is launched."""
import ctypes
import inspect
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mi355_qlinear.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from sglang_amd import _lib

    L = _lib.lib()
    declared = _declared_symbols()
    assert len(declared) >= 8
    for name in declared:
        assert getattr(L, name) is not None, name
    assert sorted(_lib.EXPORTS) == declared
    assert L.mi355_qlinear_abi_version() == _lib.ABI_VERSION == 1


def test_argument_validation_happens_before_any_device_work():
    from sglang_amd import _lib

    L = _lib.lib()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    # K not divisible by group
    rc = L.mi355_group_quant_8bit(p, _lib.BF16, p, _lib.FP8_E4M3FN, p, 4, 100, 128, 1e-10, -448.0, 448.0,
                                  _lib.QUANT_DIV, _lib.SCALE_F32, 0.0, 1, 1, None)
    assert rc == 1 and b"divisible by group" in L.mi355_last_error()
    with pytest.raises(_lib.Mi355Error, match="divisible"):
        _lib.check(rc)
    # unsupported dtype / mode / group size
    assert L.mi355_group_quant_8bit(p, _lib.I8, p, _lib.FP8_E4M3FN, p, 4, 128, 128, 1e-10, -448.0, 448.0, 0, 0, 0.0, 1, 1, None) == 1
    assert L.mi355_group_quant_8bit(p, _lib.BF16, p, _lib.F16, p, 4, 128, 128, 1e-10, -448.0, 448.0, 0, 0, 0.0, 1, 1, None) == 1
    assert L.mi355_group_quant_8bit(p, _lib.BF16, p, _lib.FP8_E4M3FN, p, 4, 128, 128, 1e-10, -448.0, 448.0, 7, 0, 0.0, 1, 1, None) == 1
    rc = L.mi355_group_quant_8bit(p, _lib.BF16, p, _lib.FP8_E4M3FN, p, 4, 96, 24, 1e-10, -448.0, 448.0, 0, 0, 0.0, 1, 1, None)
    assert rc == 2
    with pytest.raises(NotImplementedError):
        _lib.check(rc)
    # empty problem is a successful no-op and clears the message
    assert L.mi355_group_quant_8bit(None, _lib.BF16, None, _lib.FP8_E4M3FN, None, 0, 128, 128, 1e-10, -448.0, 448.0, 0, 0, 0.0, 1, 1, None) == 0
    assert L.mi355_last_error() == b""


def test_newer_entry_points_validate_before_any_device_work():
    """Every check below fails (or succeeds as an empty problem) on the host: no kernel is launched without a GPU."""
    from sglang_amd import _lib

    L = _lib.lib()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    # per-tensor quantizer: dtype, per-row scale copy only in static mode, empty tensor
    assert L.mi355_per_tensor_quant_fp8(p, _lib.I8, p, p, 16, 0, None, 0, None) == 1
    assert L.mi355_per_tensor_quant_fp8(p, _lib.BF16, p, p, 16, 0, p, 4, None) == 1 and b"static" in L.mi355_last_error()
    assert L.mi355_per_tensor_quant_fp8(p, _lib.BF16, p, None, 16, 0, None, 0, None) == 1
    assert L.mi355_per_tensor_quant_fp8(None, _lib.BF16, None, p, 0, 0, None, 0, None) == 0
    # fused activation + quantizer: fp32 input is not a 16-bit type, hidden size must be whole groups, empty problem
    assert L.mi355_silu_mul_group_quant_fp8(p, _lib.F32, p, p, 1, 4, 128, None, 0, 4, None) == 1
    assert L.mi355_silu_mul_group_quant_fp8(p, _lib.BF16, p, p, 1, 4, 100, None, 0, 4, None) == 2
    assert L.mi355_silu_mul_group_quant_fp8(None, _lib.BF16, None, None, 0, 4, 128, None, 0, 4, None) == 0
    # whole-row group quantizer: eps positive, a known mode, a float input type, rows of whole 16-byte vectors, empty tensor
    R = L.mi355_row_group_quant_fp8
    assert R(p, _lib.BF16, p, p, 4, 256, 0.0, _lib.QUANT_DIV, None) == 1 and b"eps" in L.mi355_last_error()
    assert R(p, _lib.BF16, p, p, 4, 256, 1e-10, _lib.QUANT_MUL, None) == 1 and b"mode" in L.mi355_last_error()
    assert R(p, _lib.I8, p, p, 4, 256, 1e-10, _lib.QUANT_RCP, None) == 1
    assert R(p, _lib.BF16, p, p, 4, 100, 1e-10, _lib.QUANT_RCP, None) == 2
    assert R(None, _lib.BF16, None, None, 0, 256, 1e-10, _lib.QUANT_DIV, None) == 0
    # weight-side block cast / dequant
    assert L.mi355_block_cast_to_fp8(p, _lib.I8, p, p, 128, 128, None) == 1
    assert L.mi355_block_cast_to_fp8(None, _lib.BF16, None, None, 0, 128, None) == 0
    assert L.mi355_block_dequant_fp8(p, p, p, _lib.I8, 128, 128, None) == 1
    assert L.mi355_block_dequant_fp8(None, None, None, _lib.BF16, 128, 0, None) == 0
    # UE8M0 GEMM: bias needs a 16-bit output, strides at least the row length, empty problem; workspace query is pure
    assert L.mi355_fp8_blockwise_mm_ue8m0(p, p, p, p, p, p, _lib.F32, 4, 128, 128, 128, 128, 4, 1, 128, 128, None, 0, None) == 1
    assert L.mi355_fp8_blockwise_mm_ue8m0(p, p, p, p, None, p, _lib.BF16, 4, 128, 128, 64, 128, 4, 1, 128, 128, None, 0, None) == 1
    assert L.mi355_fp8_blockwise_mm_ue8m0(p, p, p, p, None, p, _lib.BF16, 0, 128, 128, 128, 128, 4, 1, 128, 128, None, 0, None) == 0
    assert L.mi355_fp8_blockwise_mm_ue8m0_workspace_bytes(0, 128, 128) == 0
    need = L.mi355_fp8_blockwise_mm_ue8m0_workspace_bytes(4, 512, 1024)
    assert need > 0 and need % 256 == 0
    # one-call linear with the quantizer's arithmetic chosen: a known mode, K whole groups, a workspace, empty problem
    B = L.mi355_fp8_block_linear_mode
    assert B(p, _lib.BF16, _lib.QUANT_MUL, p, p, 8, 1, None, p, _lib.BF16, 4, 128, 1024, 1024, 128, p, 1 << 20, None) == 1
    assert b"quant_mode" in L.mi355_last_error()
    assert B(p, _lib.BF16, _lib.QUANT_RCP, p, p, 8, 1, None, p, _lib.BF16, 4, 128, 1000, 1000, 128, p, 1 << 20, None) == 1
    assert B(p, _lib.BF16, _lib.QUANT_RCP, p, p, 8, 1, None, p, _lib.BF16, 4, 128, 1024, 1024, 128, None, 0, None) == 4
    assert B(None, _lib.BF16, _lib.QUANT_DIV, None, None, 8, 1, None, None, _lib.BF16, 0, 128, 1024, 1024, 128, None, 0, None) == 0
    # one-call INT8 linear: output dtype, K bound, strides, workspace, empty problem
    I = L.mi355_int8_linear
    assert I(p, _lib.BF16, p, p, None, p, _lib.F32, 4, 128, 1024, 1024, 128, p, 1 << 20, None) == 1
    assert I(p, _lib.BF16, p, p, None, p, _lib.BF16, 4, 128, 1 << 17, 1 << 17, 128, p, 1 << 20, None) == 1
    assert I(p, _lib.BF16, p, p, None, p, _lib.BF16, 4, 128, 1024, 512, 128, p, 1 << 20, None) == 1
    assert I(p, _lib.BF16, p, p, None, p, _lib.BF16, 4, 128, 1024, 1024, 128, None, 0, None) == 4
    assert I(None, _lib.BF16, None, None, None, None, _lib.BF16, 0, 128, 1024, 1024, 128, None, 0, None) == 0
    assert L.mi355_int8_linear_workspace_bytes(0, 128, 1024) == 0 and L.mi355_int8_linear_workspace_bytes(4, 128, 1024) % 256 == 0
    # one-call per-token FP8 linear: output dtype, workspace, empty problem
    T = L.mi355_fp8_per_token_linear
    assert T(p, _lib.BF16, p, p, None, p, _lib.F32, 4, 128, 1024, 1024, 128, p, 1 << 20, None) == 1
    assert T(p, _lib.BF16, p, p, None, p, _lib.BF16, 4, 128, 1024, 1024, 128, None, 0, None) == 4
    assert T(p, _lib.BF16, p, p, None, p, _lib.BF16, 4, 128, 1024, 1024, 128, p, 16, None) == 4
    assert T(None, _lib.BF16, None, None, None, None, _lib.BF16, 0, 128, 1024, 1024, 128, None, 0, None) == 0
    assert L.mi355_fp8_per_token_linear_workspace_bytes(4, 128, 1024) % 256 == 0
    # one-call block-FP8 linear with packed scales: output dtype, K whole groups, workspace, empty problem
    U = L.mi355_fp8_block_linear_ue8m0
    assert U(p, _lib.BF16, p, p, 1, 128, None, p, _lib.F32, 4, 128, 1024, 1024, 128, p, 1 << 20, None) == 1
    assert U(p, _lib.BF16, p, p, 1, 128, None, p, _lib.BF16, 4, 128, 1000, 1000, 128, p, 1 << 20, None) == 1
    assert U(p, _lib.BF16, p, p, 1, 128, None, p, _lib.BF16, 4, 128, 1024, 1024, 128, None, 0, None) == 4
    assert U(None, _lib.BF16, None, None, 1, 128, None, None, _lib.BF16, 0, 128, 1024, 1024, 128, None, 0, None) == 0
    assert L.mi355_fp8_block_linear_ue8m0_workspace_bytes(4, 128, 1024) % 256 == 0
    # grouped GEMM: output dtype, K whole blocks, workspace present and large enough, empty problem; queries are pure
    G = L.mi355_fp8_blockwise_scaled_grouped_mm
    tail = (128, 128, 128 * 128, 1, 1, 1, 1, 1, 128)  # lda, ldb, expert stride, scale strides, ldo
    assert G(p, p, p, p, p, _lib.F32, p, p, 2, 8, 128, 128, *tail, p, 1 << 20, None) == 1
    assert G(p, p, p, p, p, _lib.BF16, p, p, 2, 8, 128, 100, 100, 100, 12800, 1, 1, 1, 1, 1, 128, p, 1 << 20, None) == 2
    assert G(p, p, p, p, p, _lib.BF16, None, p, 2, 8, 128, 128, *tail, p, 1 << 20, None) == 1
    assert G(p, p, p, p, p, _lib.BF16, p, p, 2, 8, 128, 128, *tail, None, 0, None) == 4 and b"workspace" in L.mi355_last_error()
    assert G(p, p, p, p, p, _lib.BF16, p, p, 2, 8, 128, 128, *tail, p, 16, None) == 4
    assert G(None, None, None, None, None, _lib.BF16, None, None, 0, 0, 128, 128, *tail, None, 0, None) == 0
    W = L.mi355_fp8_blockwise_scaled_grouped_mm_workspace_bytes
    assert W(0, 8, 128, 128) == 0 and W(2, 8, 128, 128) % 256 == 0 and W(256, 32768, 512, 7168) > W(256, 256, 512, 7168) > 0
    plan = _lib.grouped_gemm_plan(256, 32768, 512, 7168)
    assert plan["small_tile"] == "128x256" and plan["max_big_tiles"] == 32768 // 129 and plan["max_small_tiles"] == 256
    assert _lib.grouped_gemm_plan(256, 256, 512, 7168) == {
        "kernel": "grouped_pingpong+grouped_dma3", "small_tile": "64x256", "max_big_tiles": 1, "max_small_tiles": 256, "tiles_n": 2}


def test_operator_schemas_are_the_reference_ones():
    from sglang_amd import ops

    ops.register()
    ops.register()  # idempotent
    for name in ("int8_scaled_mm", "fp8_blockwise_scaled_mm", "sgl_per_token_group_quant_8bit",
                 "sgl_per_token_group_quant_8bit_v2"):
        op = getattr(torch.ops.sgl_kernel, name).default
        got = str(op._schema)
        want = "sgl_kernel::" + ops.SCHEMAS[name]
        assert got.replace(" ", "") == want.replace(" ", ""), (got, want)


def test_python_surface_matches_reference_signatures():
    from sglang_amd import fp8_kernel, sgl_kernel

    sig = inspect.signature(sgl_kernel.sgl_per_token_group_quant_8bit)
    assert list(sig.parameters) == ["input", "output_q", "output_s", "group_size", "eps", "fp8_min", "fp8_max",
                                    "scale_ue8m0", "fuse_silu_and_mul", "masked_m", "enable_v2"]
    assert sgl_kernel.sgl_per_token_group_quant_fp8 is sgl_kernel.sgl_per_token_group_quant_8bit
    assert list(inspect.signature(sgl_kernel.fp8_blockwise_scaled_mm).parameters) == [
        "mat_a", "mat_b", "scales_a", "scales_b", "out_dtype"]
    assert list(inspect.signature(sgl_kernel.int8_scaled_mm).parameters) == [
        "mat_a", "mat_b", "scales_a", "scales_b", "out_dtype", "bias"]
    sig = inspect.signature(fp8_kernel.per_token_group_quant_fp8)
    assert list(sig.parameters) == ["x", "group_size", "eps", "dtype", "column_major_scales", "scale_tma_aligned",
                                    "scale_ue8m0"]
    assert sig.parameters["eps"].default == 1e-10 and sig.parameters["dtype"].default == torch.float8_e4m3fn
    sig = inspect.signature(fp8_kernel.w8a8_block_fp8_matmul)
    assert list(sig.parameters) == ["A", "B", "As", "Bs", "block_size", "output_dtype"]
    assert sig.parameters["output_dtype"].default == torch.float16
    assert fp8_kernel.fp8_max == 448.0 and fp8_kernel.fp8_min == -448.0


def test_scale_allocator_shapes_and_strides():
    from sglang_amd.fp8_kernel import create_per_token_group_quant_fp8_output_scale as mk

    s = mk((130, 1664), "cpu", 128, False, False, False)
    assert s.shape == (130, 13) and s.is_contiguous() and s.dtype == torch.float32
    s = mk((130, 1664), "cpu", 128, True, False, False)
    assert s.shape == (130, 13) and s.stride() == (1, 130)
    s = mk((130, 1664), "cpu", 128, True, True, False)
    assert s.shape == (130, 13) and s.stride() == (1, 132)
    s = mk((130, 1664), "cpu", 128, True, True, True)
    assert s.shape == (130, 4) and s.stride() == (1, 132) and s.dtype == torch.int32
    s = mk((3, 7, 256), "cpu", 64, False, False, False)
    assert s.shape == (3, 7, 4)


def test_host_checks_reject_bad_operands_with_reference_wording():
    from sglang_amd import ops, sgl_kernel

    a = torch.zeros(4, 256, dtype=torch.float8_e4m3fn)
    # through the dispatcher a CPU tensor finds no kernel, exactly as with the reference's CUDA-only registration
    with pytest.raises(NotImplementedError, match="CPU"):
        sgl_kernel.fp8_blockwise_scaled_mm(a, a.t(), torch.zeros(4, 2), torch.zeros(2, 2), torch.bfloat16)
    # the registered host functions themselves speak the reference's TORCH_CHECK wording
    with pytest.raises(RuntimeError, match="mat_a must be a CUDA tensor"):
        ops.fp8_blockwise_scaled_mm(a, a.t(), torch.zeros(4, 2), torch.zeros(2, 2), torch.bfloat16)
    with pytest.raises(RuntimeError, match="mat_a must be a CUDA tensor"):
        ops.int8_scaled_mm(a.view(torch.int8), a.view(torch.int8).t(), torch.zeros(4), torch.zeros(4), torch.bfloat16)
    with pytest.raises(RuntimeError, match="input must be a CUDA tensor"):
        ops.sgl_per_token_group_quant_8bit(torch.zeros(4, 256), a, torch.zeros(4, 2), 128, 1e-10, -448.0, 448.0, False)
    with pytest.raises(AssertionError, match="only v2 support"):
        sgl_kernel.sgl_per_token_group_quant_8bit(torch.zeros(4, 256), a, torch.zeros(4, 2), 128, 1e-10, -448.0, 448.0,
                                                  fuse_silu_and_mul=True, enable_v2=False)
    with pytest.raises(NotImplementedError):
        ops.sgl_per_token_group_quant_8bit_v2(torch.zeros(4, 256), a, torch.zeros(4, 2), 128, 1e-10, -448.0, 448.0,
                                              False, True, None)


def test_bench_refuses_more_than_one_gpu():
    """The path is a one-GPU path: bench.py says so instead of launching ranks."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "ONE GPU" in (r.stdout + r.stderr)
