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


if __name__ == "__main__":
    main()
