"""ctypes front end of the CPU oracle (``qlinear_oracle.c``).  TEST INFRASTRUCTURE ONLY.

Nothing in the product package may import this module: it exists so that tests, the
smoke check and the benchmark's CPU-baseline leg can compare the HIP kernels with an
independent IEEE-fp32 restatement of the reference arithmetic.

All tensors here are CPU ``torch`` tensors (torch is only the container: bf16/fp8 have
no numpy dtype); every computation happens in the C library, except `per_token_row_sum`
(an fp64 torch sum).

Parity unpinned (see the functions' own notes and the header of qlinear_oracle.c): the order of
the fp32 additions inside one 128-wide K block of the FP8 GEMM, the bits of exp inside the
fused silu, and the fp32 reduction order of the row sums of per_token_quant_int8(cal_sum=True).
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional, Tuple

import torch

_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "libqlinear_oracle.so")

DT_F32, DT_F16, DT_BF16, DT_FP8, DT_I8, DT_I32 = range(6)
QUANT_DIV, QUANT_RCP, QUANT_MUL = range(3)
SCALE_F32, SCALE_UE8M0_PACKED = range(2)
EPI_COL_ROW, EPI_ROW_COL_ACC, EPI_TORCH = range(3)

_MODES = {"div": QUANT_DIV, "rcp": QUANT_RCP, "mul": QUANT_MUL}
_DT = {
    torch.float32: DT_F32,
    torch.float16: DT_F16,
    torch.bfloat16: DT_BF16,
    torch.float8_e4m3fn: DT_FP8,
    torch.int8: DT_I8,
    torch.int32: DT_I32,
}


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile beside it and return the library path."""
    src = os.path.join(_DIR, "qlinear_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _DIR, "-B", "libqlinear_oracle.so"], check=True, capture_output=True)
    return _SO


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        i64, i32, f32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p
        L.oracle_group_quant.argtypes = [vp, i32, vp, i32, vp, i64, i64, i32, f32, f32, f32, i32, i32, f32, i64, i64]
        L.oracle_group_quant.restype = i32
        L.oracle_per_token_quant_int8.argtypes = [vp, i32, vp, vp, i64, i64]
        L.oracle_per_token_quant_int8.restype = i32
        L.oracle_per_token_quant_fp8.argtypes = [vp, i32, vp, vp, i64, i64]
        L.oracle_per_token_quant_fp8.restype = i32
        L.oracle_per_tensor_quant_fp8.argtypes = [vp, i32, vp, vp, i64, i32]
        L.oracle_block_cast_to_fp8.argtypes = [vp, i32, vp, vp, i64, i64]
        L.oracle_block_cast_to_fp8.restype = i32
        L.oracle_block_dequant_fp8.argtypes = [vp, vp, vp, i32, i64, i64]
        L.oracle_block_dequant_fp8.restype = i32
        L.oracle_silu_mul.argtypes = [vp, i32, vp, i64, i64]
        L.oracle_silu_mul.restype = i32
        L.oracle_expf.argtypes = [ctypes.c_float]
        L.oracle_expf.restype = ctypes.c_float
        L.oracle_per_tensor_quant_fp8.restype = i32
        L.oracle_fp8_scaled_mm.argtypes = [vp, vp, vp, vp, vp, vp, i32, vp] + [i64] * 6
        L.oracle_fp8_scaled_mm.restype = i32
        L.oracle_fp8_blockwise_mm.argtypes = [vp, vp, vp, vp, vp, i32, vp] + [i64] * 10
        L.oracle_fp8_blockwise_mm.restype = i32
        L.oracle_int8_mm_acc.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64]
        L.oracle_int8_mm_acc.restype = i32
        L.oracle_int8_epilogue.argtypes = [vp, vp, vp, vp, vp, i32, i32, i64, i64, i64]
        L.oracle_int8_epilogue.restype = i32
        L.oracle_e4m3fn_encode.argtypes = [f32]
        L.oracle_e4m3fn_encode.restype = ctypes.c_uint8
        L.oracle_e4m3fn_decode.argtypes = [ctypes.c_uint8]
        L.oracle_e4m3fn_decode.restype = f32
        L.oracle_f32_to_bf16.argtypes = [f32]
        L.oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.oracle_f32_to_f16.argtypes = [f32]
        L.oracle_f32_to_f16.restype = ctypes.c_uint16
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f16_to_f32.restype = f32
        L.oracle_num_threads.restype = i32
        L.oracle_set_num_threads.argtypes = [i32]
        _lib = L
    return _lib


def num_threads() -> int:
    return lib().oracle_num_threads()


def set_num_threads(n: int) -> None:
    lib().oracle_set_num_threads(int(n))


def _cpu(t: torch.Tensor) -> torch.Tensor:
    assert t.device.type == "cpu", "the oracle works on host tensors"
    return t


def _align(x: int, a: int) -> int:
    return (x + a - 1) // a * a


def make_scale_tensor(M: int, K: int, group: int, layout: str) -> torch.Tensor:
    """Scale tensor with the strides the reference's allocator produces
    (python/sglang/srt/layers/quantization/fp8_kernel.py:433-474), for a 2-D input.

    layout: "row"          fp32 [M, K/g] contiguous                       (:469-474)
            "col"          fp32 [M, K/g] with strides (1, M)              (:463-468)
            "col_aligned"  fp32 [M, K/g] with strides (1, align4(M))      (:454-462)
            "ue8m0"        int32 [M, align4(K/128)/4] strides (1, align4(M))  (:441-452)
    """
    G = K // group
    if layout == "row":
        return torch.zeros(M, G, dtype=torch.float32)
    if layout == "col":
        return torch.zeros(G, M, dtype=torch.float32).permute(-1, -2)
    if layout == "col_aligned":
        return torch.zeros(G, _align(M, 4), dtype=torch.float32).transpose(-1, -2)[:M, :]
    if layout == "ue8m0":
        assert group == 128
        return torch.zeros(_align(G, 4) // 4, _align(M, 4), dtype=torch.int32).transpose(-1, -2)[:M, :]
    raise ValueError(layout)


def group_quant(
    x: torch.Tensor,
    group: int,
    mode: str = "div",
    layout: str = "row",
    dst_dtype: torch.dtype = torch.float8_e4m3fn,
    eps: float = 1e-10,
    pow2_floor: float = 0.0,
    qmin: Optional[float] = None,
    qmax: Optional[float] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-token-group quantization of a contiguous 2-D tensor; returns (q, s)."""
    x = _cpu(x)
    assert x.dim() == 2 and x.is_contiguous()
    M, K = x.shape
    if qmax is None:
        qmax = 448.0 if dst_dtype == torch.float8_e4m3fn else 127.0
    if qmin is None:
        qmin = -448.0 if dst_dtype == torch.float8_e4m3fn else -128.0
    q = torch.zeros(M, K, dtype=torch.uint8).view(dst_dtype)
    s = make_scale_tensor(M, K, group, layout)
    kind = SCALE_UE8M0_PACKED if layout == "ue8m0" else SCALE_F32
    rc = lib().oracle_group_quant(
        x.data_ptr(), _DT[x.dtype], q.data_ptr(), _DT[dst_dtype], s.data_ptr(), M, K, group,
        eps, qmin, qmax, _MODES[mode], kind, pow2_floor, s.stride(0), s.stride(1),
    )
    assert rc == 0, f"oracle_group_quant failed: {rc}"
    return q, s


def unpack_ue8m0(s_packed: torch.Tensor, G: int) -> torch.Tensor:
    """int32 [M, ceil(G/4)] packed exponent bytes (any strides) -> uint8 [M, G]."""
    M = s_packed.shape[0]
    dense = torch.empty(tuple(s_packed.shape), dtype=torch.int32)  # fresh row-major storage whatever the strides
    dense.copy_(s_packed)
    b = dense.view(torch.uint8).reshape(M, -1)  # little endian: byte j of word w = group 4w+j
    return b[:, :G].contiguous()


def per_token_quant_int8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    x = _cpu(x)
    assert x.dim() == 2 and x.is_contiguous()
    M, K = x.shape
    q = torch.zeros(M, K, dtype=torch.int8)
    s = torch.zeros(M, 1, dtype=torch.float32)
    rc = lib().oracle_per_token_quant_int8(x.data_ptr(), _DT[x.dtype], q.data_ptr(), s.data_ptr(), M, K)
    assert rc == 0
    return q, s


def per_token_row_sum(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Row sums of per_token_quant_int8(cal_sum=True) (python/sglang/srt/layers/quantization/int8_kernel.py:52-54): the
    exact sum of the row (fp64), the sum of magnitudes, and the exact sum rounded to the input's type.
    PARITY UNPINNED at bit level: the reference adds in fp32 in whatever order Triton's tl.sum emits, so a conforming
    result lies within fp32 reassociation error of the exact sum before the final rounding; tests bound it by that."""
    x = _cpu(x)
    exact = x.double().sum(-1)
    return exact, x.double().abs().sum(-1), exact.to(x.dtype)


def per_token_quant_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """x [M,K] -> (e4m3fn [M,K], fp32 scales [M,1]); scale = max|x| / 448, zero rows give scale 0 and zeros."""
    x = _cpu(x)
    assert x.dim() == 2 and x.is_contiguous()
    M, K = x.shape
    q = torch.zeros(M, K, dtype=torch.uint8)
    s = torch.zeros(M, 1, dtype=torch.float32)
    rc = lib().oracle_per_token_quant_fp8(x.data_ptr(), _DT[x.dtype], q.data_ptr(), s.data_ptr(), M, K)
    assert rc == 0
    return q.view(torch.float8_e4m3fn), s


def block_cast_to_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """x [m,n] -> (e4m3fn [m,n], fp32 power-of-two scales [ceil(m/128), ceil(n/128)])."""
    x = _cpu(x).contiguous()
    m, n = x.shape
    q = torch.zeros(m, n, dtype=torch.uint8)
    s = torch.zeros((m + 127) // 128, (n + 127) // 128, dtype=torch.float32)
    rc = lib().oracle_block_cast_to_fp8(x.data_ptr(), _DT[x.dtype], q.data_ptr(), s.data_ptr(), m, n)
    assert rc == 0
    return q.view(torch.float8_e4m3fn), s


def block_dequant_fp8(q: torch.Tensor, s: torch.Tensor, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    q, s = _cpu(q).contiguous(), _cpu(s).contiguous().to(torch.float32)
    n, k = q.shape
    out = torch.zeros(n, k, dtype=dtype)
    rc = lib().oracle_block_dequant_fp8(q.view(torch.uint8).data_ptr(), s.data_ptr(), out.data_ptr(), _DT[dtype], n, k)
    assert rc == 0
    return out


def silu_mul(x: torch.Tensor) -> torch.Tensor:
    """x [..., 2H] bf16/fp16 -> [..., H] of the same dtype: T(silu(gate)) * up with the roundings of the v2 quantizer."""
    x = _cpu(x).contiguous()
    H = x.shape[-1] // 2
    out = torch.zeros(*x.shape[:-1], H, dtype=x.dtype)
    rc = lib().oracle_silu_mul(x.data_ptr(), _DT[x.dtype], out.data_ptr(), x.numel() // (2 * H), H)
    assert rc == 0
    return out


def expf(v: float) -> float:
    return float(lib().oracle_expf(float(v)))


def per_tensor_quant_fp8(x: torch.Tensor, scale: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """x (any shape) -> (e4m3fn like x, fp32 scale [1]); scale = max|x| / 448 unless given (static)."""
    x = _cpu(x).contiguous()
    q = torch.zeros(x.shape, dtype=torch.uint8)
    s = torch.zeros(1, dtype=torch.float32) if scale is None else _cpu(scale).reshape(1).to(torch.float32).clone()
    rc = lib().oracle_per_tensor_quant_fp8(x.data_ptr(), _DT[x.dtype], q.data_ptr(), s.data_ptr(), x.numel(), int(scale is not None))
    assert rc == 0
    return q.view(torch.float8_e4m3fn), s


def fp8_scaled_mm(a, w, sa, sb, out_dtype=torch.bfloat16, bias: Optional[torch.Tensor] = None, want_abs: bool = False):
    """a [M,K] fp8, w [N,K] fp8 (weight as stored), sa [M], sb [N], bias [N] in the output dtype or None ->
    out [M,N] = cast(sa[m] * (sb[n] * sum_k a*w) + bias[n]); with want_abs also the fp32 magnitude matrix."""
    a, w, sa, sb = _cpu(a), _cpu(w), _cpu(sa).reshape(-1), _cpu(sb).reshape(-1)
    M, K = a.shape
    N = w.shape[0]
    assert w.shape[1] == K and a.stride(1) == 1 and w.stride(1) == 1 and sa.numel() == M and sb.numel() == N
    if bias is not None:
        bias = _cpu(bias)
        assert bias.dtype == out_dtype and bias.numel() == N
    out = torch.zeros(M, N, dtype=out_dtype)
    ab = torch.zeros(M, N, dtype=torch.float32) if want_abs else None
    rc = lib().oracle_fp8_scaled_mm(
        a.data_ptr(), w.data_ptr(), sa.data_ptr(), sb.data_ptr(), bias.data_ptr() if bias is not None else None,
        out.data_ptr(), _DT[out_dtype], ab.data_ptr() if want_abs else None, M, N, K, a.stride(0), w.stride(0), out.stride(0))
    assert rc == 0
    return (out, ab) if want_abs else out


def fp8_blockwise_mm(
    a: torch.Tensor,
    w: torch.Tensor,
    sa: torch.Tensor,
    sw: torch.Tensor,
    out_dtype: torch.dtype = torch.bfloat16,
    want_abs: bool = False,
):
    """a [M,K] fp8, w [N,K] fp8 (weight as stored), sa [M, ceil(K/128)], sw [ceil(N/128), ceil(K/128)]
    (any strides) -> out [M,N]; with want_abs also the fp32 magnitude matrix."""
    a, w, sa, sw = _cpu(a), _cpu(w), _cpu(sa), _cpu(sw)
    M, K = a.shape
    N, K2 = w.shape
    assert K == K2 and a.stride(1) == 1 and w.stride(1) == 1
    KB = (K + 127) // 128
    assert tuple(sa.shape) == (M, KB), (sa.shape, (M, KB))
    assert tuple(sw.shape) == ((N + 127) // 128, KB), (sw.shape, N, KB)
    assert sa.dtype == torch.float32 and sw.dtype == torch.float32
    out = torch.zeros(M, N, dtype=out_dtype)
    ab = torch.zeros(M, N, dtype=torch.float32) if want_abs else None
    rc = lib().oracle_fp8_blockwise_mm(
        a.data_ptr(), w.data_ptr(), sa.data_ptr(), sw.data_ptr(), out.data_ptr(), _DT[out_dtype],
        ab.data_ptr() if want_abs else None, M, N, K, a.stride(0), w.stride(0),
        sa.stride(0), sa.stride(1), sw.stride(0), sw.stride(1), out.stride(0),
    )
    assert rc == 0
    return (out, ab) if want_abs else out


def int8_mm_acc(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """a [M,K] int8, w [N,K] int8 (weight as stored) -> exact int32 [M,N]."""
    a, w = _cpu(a), _cpu(w)
    M, K = a.shape
    N = w.shape[0]
    assert w.shape[1] == K and a.stride(1) == 1 and w.stride(1) == 1
    acc = torch.zeros(M, N, dtype=torch.int32)
    rc = lib().oracle_int8_mm_acc(a.data_ptr(), w.data_ptr(), acc.data_ptr(), M, N, K, a.stride(0), w.stride(0))
    assert rc == 0
    return acc


def int8_epilogue(
    acc: torch.Tensor,
    sa: torch.Tensor,
    sb: torch.Tensor,
    out_dtype: torch.dtype,
    bias: Optional[torch.Tensor] = None,
    order: int = EPI_COL_ROW,
) -> torch.Tensor:
    acc = _cpu(acc).contiguous()
    M, N = acc.shape
    sa = _cpu(sa).contiguous().view(-1)
    sb = _cpu(sb).contiguous().view(-1)
    assert sa.numel() == M and sb.numel() == N
    if bias is not None:
        bias = _cpu(bias).contiguous()
        assert bias.dtype == out_dtype and bias.numel() == N
    out = torch.zeros(M, N, dtype=out_dtype)
    rc = lib().oracle_int8_epilogue(
        acc.data_ptr(), sa.data_ptr(), sb.data_ptr(), bias.data_ptr() if bias is not None else None,
        out.data_ptr(), _DT[out_dtype], order, M, N, out.stride(0),
    )
    assert rc == 0
    return out


def int8_scaled_mm(a, w, sa, sb, out_dtype, bias=None, order: int = EPI_COL_ROW) -> torch.Tensor:
    return int8_epilogue(int8_mm_acc(a, w), sa, sb, out_dtype, bias, order)


def _batch(fn_name: str, src: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    src = _cpu(src).contiguous()
    out = torch.zeros(src.numel(), dtype=out_dtype)
    fn = getattr(lib(), fn_name)
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
    fn.restype = None
    fn(src.data_ptr(), out.data_ptr(), src.numel())
    return out.reshape(src.shape)


def e4m3fn_encode(x: torch.Tensor) -> torch.Tensor:
    """fp32 tensor -> uint8 e4m3fn codes."""
    return _batch("oracle_e4m3fn_encode_n", x.to(torch.float32), torch.uint8)


def e4m3fn_decode(b: torch.Tensor) -> torch.Tensor:
    return _batch("oracle_e4m3fn_decode_n", b, torch.float32)


def f32_to_bf16_bits(x: torch.Tensor) -> torch.Tensor:
    return _batch("oracle_f32_to_bf16_n", x, torch.int16)


def f32_to_f16_bits(x: torch.Tensor) -> torch.Tensor:
    return _batch("oracle_f32_to_f16_n", x, torch.int16)


def f16_bits_to_f32(b: torch.Tensor) -> torch.Tensor:
    return _batch("oracle_f16_to_f32_n", b, torch.float32)
