"""Golden fixtures (tests/golden/qlinear_golden.npz, written by tests/golden/make_golden.py).

CPU: the oracle must still reproduce them (guards the checker itself against regressions).
GPU: the HIP kernels must reproduce them without the oracle in the loop."""
import os

import numpy as np
import pytest
import torch

from fp8_tolerance import check_fp8_gemm, magnitudes

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "qlinear_golden.npz")
FP8 = torch.float8_e4m3fn


@pytest.fixture(scope="module")
def gold():
    z = np.load(GOLD, allow_pickle=False)
    return {k: torch.from_numpy(z[k].copy()) for k in z.files}


def _bf16(t):
    return t.view(torch.bfloat16)


def _f32(t):
    return t.view(torch.float32)


def _dequant_rows(q_u8, s_f32):
    """codes [R, K] with one scale per 128-wide K group [R, K/128] -> fp32 (the fixtures hold no sum of magnitudes; it is
    formed here from their operands with plain torch, without the oracle)."""
    return q_u8.view(FP8).float() * s_f32.repeat_interleave(128, dim=1)[:, : q_u8.shape[1]]


def _dequant_blocks(q_u8, s_f32):
    """codes [N, K] with one scale per 128 x 128 block [N/128, K/128] -> fp32."""
    n, k = q_u8.shape
    return q_u8.view(FP8).float() * s_f32.repeat_interleave(128, dim=0)[:n].repeat_interleave(128, dim=1)[:, :k]


def test_oracle_reproduces_quant_fixtures(oracle, gold):
    x = _bf16(gold["quant_x_bf16"])
    for mode, floor in (("div", 1e-10), ("rcp", 0.0), ("mul", 0.0)):
        q, s = oracle.group_quant(x, 128, mode=mode)
        assert torch.equal(q.view(torch.uint8), gold[f"quant_{mode}_q"])
        assert torch.equal(s.view(torch.int32), gold[f"quant_{mode}_s_f32"])
        q, s = oracle.group_quant(x, 128, mode=mode, layout="ue8m0", pow2_floor=floor)
        assert torch.equal(q.view(torch.uint8), gold[f"quant_{mode}_ue8m0_q"])
        assert torch.equal(oracle.unpack_ue8m0(s, 4), gold[f"quant_{mode}_ue8m0_bytes"])
    q, s = oracle.group_quant(x, 128, mode="div", dst_dtype=torch.int8)
    assert torch.equal(q, gold["quant_div_int8_q"]) and torch.equal(s.view(torch.int32), gold["quant_div_int8_s_f32"])
    pq, ps = oracle.per_token_quant_int8(x)
    assert torch.equal(pq, gold["ptq_q"]) and torch.equal(ps.view(torch.int32), gold["ptq_s_f32"])


def test_oracle_reproduces_gemm_fixtures(oracle, gold):
    aq, asc = gold["gemm_a_q"].view(FP8), _f32(gold["gemm_a_s_f32"])
    wq, ws = gold["gemm_w_q"].view(FP8), _f32(gold["gemm_w_s_f32"])
    assert torch.equal(oracle.fp8_blockwise_mm(aq, wq, asc, ws, torch.float32).view(torch.int32), gold["gemm_out_f32"])
    assert torch.equal(oracle.fp8_blockwise_mm(aq, wq, asc, ws, torch.bfloat16).view(torch.int16), gold["gemm_out_bf16"])
    acc = oracle.int8_mm_acc(gold["int8_a"], gold["int8_w"])
    assert torch.equal(acc, gold["int8_acc"])
    out = oracle.int8_epilogue(acc, _f32(gold["int8_sa_f32"]), _f32(gold["int8_sb_f32"]), torch.bfloat16,
                               _bf16(gold["int8_bias_bf16"]))
    assert torch.equal(out.view(torch.int16), gold["int8_out_bf16"])


@pytest.mark.gpu
def test_gpu_reproduces_quant_fixtures(gpu, gold):
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8, sglang_per_token_group_quant_8bit
    from sglang_amd.int8_kernel import per_token_quant_int8

    x = _bf16(gold["quant_x_bf16"]).to(gpu)
    q, s = per_token_group_quant_fp8(x, 128)  # Triton row-major arithmetic: x * (1/s)
    assert torch.equal(q.cpu().view(torch.uint8), gold["quant_rcp_q"])
    assert torch.equal(s.cpu().view(torch.int32), gold["quant_rcp_s_f32"])
    for v2, mode in ((False, "div"), (True, "mul")):
        q, s = sglang_per_token_group_quant_8bit(x, 128, FP8, enable_v2=v2)
        assert torch.equal(q.cpu().view(torch.uint8), gold[f"quant_{mode}_q"])
        assert torch.equal(s.cpu().view(torch.int32), gold[f"quant_{mode}_s_f32"])
        q, s = sglang_per_token_group_quant_8bit(x, 128, FP8, column_major_scales=True, scale_tma_aligned=True,
                                                 scale_ue8m0=True, enable_v2=v2)
        assert torch.equal(q.cpu().view(torch.uint8), gold[f"quant_{mode}_ue8m0_q"])
        dense = torch.empty(tuple(s.shape), dtype=torch.int32)
        dense.copy_(s.cpu())
        assert torch.equal(dense.view(torch.uint8).reshape(s.shape[0], -1)[:, :4], gold[f"quant_{mode}_ue8m0_bytes"])
    q, s = sglang_per_token_group_quant_8bit(x, 128, torch.int8, enable_v2=False)
    assert torch.equal(q.cpu(), gold["quant_div_int8_q"]) and torch.equal(s.cpu().view(torch.int32), gold["quant_div_int8_s_f32"])
    pq, ps = per_token_quant_int8(x)
    assert torch.equal(pq.cpu(), gold["ptq_q"]) and torch.equal(ps.cpu().view(torch.int32), gold["ptq_s_f32"])


@pytest.mark.gpu
def test_gpu_reproduces_gemm_fixtures(gpu, gold):
    from sglang_amd import ops
    from sglang_amd.fp8_kernel import w8a8_block_fp8_matmul
    from sglang_amd.sgl_kernel import int8_scaled_mm

    aq, asc = gold["gemm_a_q"].view(FP8).to(gpu), _f32(gold["gemm_a_s_f32"]).to(gpu)
    wq, ws = gold["gemm_w_q"].view(FP8).to(gpu), _f32(gold["gemm_w_s_f32"]).to(gpu)
    ref = _f32(gold["gemm_out_f32"])
    out = w8a8_block_fp8_matmul(aq, wq, asc, ws, [128, 128], torch.float32)
    mag = magnitudes(_dequant_rows(gold["gemm_a_q"], _f32(gold["gemm_a_s_f32"])), _dequant_blocks(gold["gemm_w_q"], _f32(gold["gemm_w_s_f32"])))
    check_fp8_gemm(out, ref, mag, "gemm fixture")
    a, w = gold["int8_a"].to(gpu), gold["int8_w"].to(gpu)
    assert torch.equal(ops.int8_mm_raw_accumulators(a, w.t()).cpu(), gold["int8_acc"])
    out = int8_scaled_mm(a, w.t(), _f32(gold["int8_sa_f32"]).to(gpu), _f32(gold["int8_sb_f32"]).to(gpu), torch.bfloat16,
                         _bf16(gold["int8_bias_bf16"]).to(gpu))
    assert torch.equal(out.cpu().view(torch.int16), gold["int8_out_bf16"])


# ---- the quantizers and GEMMs around the first three (tests/golden/qlinear_golden_more.npz)

MORE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "qlinear_golden_more.npz")


@pytest.fixture(scope="module")
def more():
    z = np.load(MORE, allow_pickle=False)
    return {k: torch.from_numpy(z[k].copy()) for k in z.files}


def test_oracle_reproduces_the_other_fixtures(oracle, more):
    x = _bf16(more["x_bf16"])
    q, s = oracle.per_token_quant_fp8(x)
    assert torch.equal(q.view(torch.uint8), more["ptq_fp8_q"]) and torch.equal(s.view(torch.int32), more["ptq_fp8_s_f32"])
    q, s = oracle.per_tensor_quant_fp8(x)
    assert torch.equal(q.view(torch.uint8), more["pt_dyn_q"]) and torch.equal(s.view(torch.int32), more["pt_dyn_s_f32"])
    q, _ = oracle.per_tensor_quant_fp8(x, _f32(more["pt_static_scale_f32"]))
    assert torch.equal(q.view(torch.uint8), more["pt_static_q"])
    v = oracle.silu_mul(_bf16(more["silu_in_bf16"]))
    assert torch.equal(v.view(torch.int16), more["silu_v_bf16"])
    q, s = oracle.group_quant(v, 128, mode="mul", layout="ue8m0")
    assert torch.equal(q.view(torch.uint8), more["silu_q"]) and torch.equal(oracle.unpack_ue8m0(s, 2), more["silu_bytes"])
    wq, ws = oracle.block_cast_to_fp8(_bf16(more["cast_w_bf16"]))
    assert torch.equal(wq.view(torch.uint8), more["cast_q"]) and torch.equal(ws.view(torch.int32), more["cast_s_f32"])
    assert torch.equal(oracle.block_dequant_fp8(wq, ws, torch.bfloat16).view(torch.int16), more["cast_back_bf16"])
    out = oracle.fp8_scaled_mm(more["ptq_fp8_q"].view(FP8), more["smm_w_q"].view(FP8), _f32(more["ptq_fp8_s_f32"]).reshape(-1),
                               _f32(more["smm_sb_f32"]), torch.float32, None)
    assert torch.equal(out.view(torch.int32), more["smm_out_f32"])
    gq, gs = more["grp_a_q"].view(FP8), _f32(more["grp_a_s_f32"])
    for e, (r0, m) in enumerate(zip(more["grp_offsets"].tolist(), more["grp_sizes"][:, 0].tolist())):
        if m:
            ref = oracle.fp8_blockwise_mm(gq[r0:r0 + m], more["grp_w_q"].view(FP8)[e], gs[r0:r0 + m], _f32(more["grp_w_s_f32"])[e],
                                          torch.float32)
            assert torch.equal(ref.view(torch.int32), more["grp_out_f32"][r0:r0 + m])


@pytest.mark.gpu
def test_gpu_reproduces_the_other_fixtures(gpu, more):
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8, sglang_per_token_quant_fp8
    from sglang_amd.fp8_utils import block_quant_dequant, per_block_cast_to_fp8
    from sglang_amd.sgl_kernel import es_fp8_blockwise_scaled_grouped_mm, fp8_scaled_mm, sgl_per_tensor_quant_fp8

    x = _bf16(more["x_bf16"]).to(gpu)
    q, s = sglang_per_token_quant_fp8(x)
    assert torch.equal(q.cpu().view(torch.uint8), more["ptq_fp8_q"]) and torch.equal(s.cpu().view(torch.int32), more["ptq_fp8_s_f32"])
    q = torch.empty_like(x, dtype=FP8)
    s = torch.zeros(1, dtype=torch.float32, device=gpu)
    sgl_per_tensor_quant_fp8(x, q, s, False)
    assert torch.equal(q.cpu().view(torch.uint8), more["pt_dyn_q"]) and torch.equal(s.cpu().view(torch.int32), more["pt_dyn_s_f32"])
    sgl_per_tensor_quant_fp8(x, q, _f32(more["pt_static_scale_f32"]).to(gpu), True)
    assert torch.equal(q.cpu().view(torch.uint8), more["pt_static_q"])
    q, s = sglang_per_token_group_quant_fp8(_bf16(more["silu_in_bf16"]).to(gpu), 128, column_major_scales=True, scale_tma_aligned=True,
                                            scale_ue8m0=True, fuse_silu_and_mul=True, enable_v2=True)
    assert torch.equal(q.cpu().view(torch.uint8), more["silu_q"])
    dense = torch.empty(tuple(s.shape), dtype=torch.int32)
    dense.copy_(s.cpu())
    assert torch.equal(dense.view(torch.uint8).reshape(s.shape[0], -1)[:, :2], more["silu_bytes"])
    wq, ws = per_block_cast_to_fp8(_bf16(more["cast_w_bf16"]).to(gpu))
    assert torch.equal(wq.cpu().view(torch.uint8), more["cast_q"]) and torch.equal(ws.cpu().view(torch.int32), more["cast_s_f32"])
    back = block_quant_dequant(wq, ws, [128, 128], torch.bfloat16)
    assert torch.equal(back.cpu().view(torch.int16), more["cast_back_bf16"])
    ref = _f32(more["smm_out_f32"])
    out = fp8_scaled_mm(more["ptq_fp8_q"].view(FP8).to(gpu), more["smm_w_q"].view(FP8).to(gpu).t(), _f32(more["ptq_fp8_s_f32"]).to(gpu),
                        _f32(more["smm_sb_f32"]).to(gpu), torch.bfloat16, None)
    mag = magnitudes(more["ptq_fp8_q"].view(FP8).float() * _f32(more["ptq_fp8_s_f32"]).reshape(-1, 1),
                     more["smm_w_q"].view(FP8).float() * _f32(more["smm_sb_f32"]).reshape(-1, 1))
    check_fp8_gemm(out, ref, mag, "fp8_scaled_mm fixture")
    E, T, N, K = 3, 9, 128, 256
    outg = torch.full((T, N), 7.0, dtype=torch.bfloat16, device=gpu)
    strides = torch.full((E,), K, dtype=torch.int64, device=gpu)
    es_fp8_blockwise_scaled_grouped_mm(
        outg, more["grp_a_q"].view(FP8).to(gpu), more["grp_w_q"].view(FP8).to(gpu).transpose(1, 2), _f32(more["grp_a_s_f32"]).to(gpu),
        _f32(more["grp_w_s_f32"]).to(gpu).transpose(1, 2), strides, strides, strides, more["grp_sizes"].to(gpu),
        more["grp_offsets"].to(gpu), torch.empty(1 << 20, dtype=torch.uint8, device=gpu))
    ref = _f32(more["grp_out_f32"])
    got = outg.float().cpu()
    ga = _dequant_rows(more["grp_a_q"], _f32(more["grp_a_s_f32"]))
    for e, (r0, m) in enumerate(zip(more["grp_offsets"].tolist(), more["grp_sizes"][:, 0].tolist())):
        if m:
            mag = magnitudes(ga[r0:r0 + m], _dequant_blocks(more["grp_w_q"][e], _f32(more["grp_w_s_f32"])[e]))
            check_fp8_gemm(got[r0:r0 + m], ref[r0:r0 + m], mag, f"grouped fixture, expert {e}")
