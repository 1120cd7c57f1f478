"""Writes the golden fixtures of this directory from the CPU oracle (run: python tests/golden/make_golden.py).

The reference stores no vectors for this path (its tests regenerate seeded random data), so these
fixtures are small seeded inputs with the outputs of the oracle, which tests/test_oracle_*.py pin against
torch's CPU routines and the reference's known-answer construction.  They guard the oracle against
regressions (CPU suite) and give the GPU suite inputs/outputs that do not depend on the oracle being built.
Everything is stored as integer arrays (bit patterns) in one compressed .npz of a few tens of KB.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import oracle  # noqa: E402
from sglang_amd.workloads import block_cast_to_fp8, make_activation, make_int8_activation, make_int8_weight  # noqa: E402


def bits(t):
    t = t.contiguous() if t.is_contiguous() else t.clone(memory_format=torch.contiguous_format)
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy()
    if t.dtype == torch.float32:
        return t.view(torch.int32).numpy()
    if t.dtype == torch.float8_e4m3fn:
        return t.view(torch.uint8).numpy()
    return t.numpy()


def main():
    out = {}
    # group quantizer: 12 x 512 bf16 with outliers and zero groups
    x = make_activation(12, 512, seed=2024, zero_group_frac=0.1, outlier_frac=0.01)
    out["quant_x_bf16"] = bits(x)
    for mode, floor in (("div", 1e-10), ("rcp", 0.0), ("mul", 0.0)):
        q, s = oracle.group_quant(x, 128, mode=mode, layout="row")
        out[f"quant_{mode}_q"], out[f"quant_{mode}_s_f32"] = bits(q), bits(s)
        q, s = oracle.group_quant(x, 128, mode=mode, layout="ue8m0", pow2_floor=floor)
        out[f"quant_{mode}_ue8m0_q"] = bits(q)
        out[f"quant_{mode}_ue8m0_bytes"] = oracle.unpack_ue8m0(s, 4).numpy()
    q, s = oracle.group_quant(x, 128, mode="div", dst_dtype=torch.int8)
    out["quant_div_int8_q"], out["quant_div_int8_s_f32"] = bits(q), bits(s)
    # blockwise FP8 GEMM: M=6, N=200 (ragged), K=384
    g = torch.Generator().manual_seed(7)
    a = make_activation(6, 384, seed=5)
    aq, asc = oracle.group_quant(a, 128, mode="div")
    wq, ws = block_cast_to_fp8(torch.randn(200, 384, generator=g) * 0.02)
    out["gemm_a_q"], out["gemm_a_s_f32"] = bits(aq), bits(asc)
    out["gemm_w_q"], out["gemm_w_s_f32"] = bits(wq), bits(ws)
    out["gemm_out_f32"] = bits(oracle.fp8_blockwise_mm(aq, wq, asc, ws, torch.float32))
    out["gemm_out_bf16"] = bits(oracle.fp8_blockwise_mm(aq, wq, asc, ws, torch.bfloat16))
    # INT8 GEMM: M=5, N=72, K=256 with bias
    ia, isa = make_int8_activation(5, 256, seed=11)
    iw, isb = make_int8_weight(72, 256, seed=12)
    bias = (torch.randn(72, generator=g) * 3).to(torch.bfloat16)
    acc = oracle.int8_mm_acc(ia, iw)
    out["int8_a"], out["int8_sa_f32"], out["int8_w"], out["int8_sb_f32"] = bits(ia), bits(isa), bits(iw), bits(isb)
    out["int8_bias_bf16"], out["int8_acc"] = bits(bias), bits(acc)
    out["int8_out_bf16"] = bits(oracle.int8_epilogue(acc, isa, isb, torch.bfloat16, bias))
    # per-token int8 quant of the quantizer input
    pq, ps = oracle.per_token_quant_int8(x)
    out["ptq_q"], out["ptq_s_f32"] = bits(pq), bits(ps)
    path = os.path.join(HERE, "qlinear_golden.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")
    write_more()


def write_more():
    """qlinear_golden_more.npz: the quantizers and GEMMs around the first three (per-token and per-tensor FP8, silu * up
    in front of the group quantizer, weight block cast, per-token x per-channel FP8 GEMM, grouped GEMM)."""
    out = {}
    g = torch.Generator().manual_seed(31)
    x = make_activation(9, 384, seed=77, outlier_frac=0.01)
    x[3] = 0
    out["x_bf16"] = bits(x)
    q, s = oracle.per_token_quant_fp8(x)
    out["ptq_fp8_q"], out["ptq_fp8_s_f32"] = bits(q), bits(s)
    q, s = oracle.per_tensor_quant_fp8(x)
    out["pt_dyn_q"], out["pt_dyn_s_f32"] = bits(q), bits(s)
    given = torch.tensor([0.0371], dtype=torch.float32)
    q, _ = oracle.per_tensor_quant_fp8(x, given)
    out["pt_static_scale_f32"], out["pt_static_q"] = bits(given), bits(q)
    # silu(gate) * up, then the v2 group quantizer with packed power-of-two scales: [7, 2 x 256]
    gu = make_activation(7, 512, seed=78, outlier_frac=0.02)
    v = oracle.silu_mul(gu)
    q, s = oracle.group_quant(v, 128, mode="mul", layout="ue8m0")
    out["silu_in_bf16"], out["silu_v_bf16"], out["silu_q"] = bits(gu), bits(v), bits(q)
    out["silu_bytes"] = oracle.unpack_ue8m0(s, 2).numpy()
    # 128 x 128 block cast of a weight [130, 200] and its inverse
    w = (torch.randn(130, 200, generator=g) * 0.02).to(torch.bfloat16)
    wq, ws = oracle.block_cast_to_fp8(w)
    out["cast_w_bf16"], out["cast_q"], out["cast_s_f32"] = bits(w), bits(wq), bits(ws)
    out["cast_back_bf16"] = bits(oracle.block_dequant_fp8(wq, ws, torch.bfloat16))
    # per-token x per-channel FP8 GEMM with bias: M=9, N=72, K=384
    aq, asc = oracle.per_token_quant_fp8(x)
    bq = ((torch.rand(72, 384, generator=g) - 0.5) * 200).to(torch.float8_e4m3fn)
    sb = torch.rand(72, generator=g) * 1e-2 + 1e-3
    bias = torch.randn(72, generator=g).to(torch.bfloat16)
    out["smm_w_q"], out["smm_sb_f32"], out["smm_bias_bf16"] = bits(bq), bits(sb), bits(bias)
    out["smm_out_f32"] = bits(oracle.fp8_scaled_mm(aq, bq, asc.reshape(-1), sb, torch.float32, None))
    # grouped GEMM: 3 experts with 5, 0 and 4 of 9 rows, N=128, K=256
    xg = make_activation(9, 256, seed=79)
    gq, gs = oracle.group_quant(xg, 128, mode="div")
    ew = ((torch.rand(3, 128, 256, generator=g) - 0.5) * 200).to(torch.float8_e4m3fn)
    es = torch.rand(3, 1, 2, generator=g) * 1e-2 + 1e-3
    rows = [(0, 5), (5, 0), (5, 4)]
    ref = torch.zeros(9, 128)
    for e, (r0, m) in enumerate(rows):
        if m:
            ref[r0:r0 + m] = oracle.fp8_blockwise_mm(gq[r0:r0 + m], ew[e], gs[r0:r0 + m], es[e], torch.float32)
    out["grp_a_q"], out["grp_a_s_f32"], out["grp_w_q"], out["grp_w_s_f32"] = bits(gq), bits(gs), bits(ew), bits(es)
    out["grp_sizes"] = np.array([[m, 128, 256] for _, m in rows], dtype=np.int32)
    out["grp_offsets"] = np.array([r0 for r0, _ in rows], dtype=np.int32)
    out["grp_out_f32"] = bits(ref)
    path = os.path.join(HERE, "qlinear_golden_more.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
