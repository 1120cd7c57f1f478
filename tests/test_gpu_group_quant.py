"""GPU parity of the per-token-group quantizer: the HIP kernel, called through the C ABI by the
reference-named Python entry points, against the CPU oracle on identical seeded inputs.
Codes and scales must match bit for bit in every rounding mode and scale layout."""
import pytest
import torch

from sglang_amd.workloads import make_activation

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def _u8(t):
    return t.view(torch.uint8)


def _same_bits(a, b):
    a, b = a.cpu(), b.cpu()
    if a.dtype in (torch.float32,):
        return torch.equal(a.view(torch.int32), b.view(torch.int32))
    if a.dtype in (FP8, torch.int8):
        return torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    return torch.equal(a, b)


def _diff_report(a, b):
    a8, b8 = _u8(a.cpu()).to(torch.int16), _u8(b.cpu()).to(torch.int16)
    d = a8 != b8
    idx = d.nonzero()[:5].tolist()
    return f"{int(d.sum())} of {d.numel()} codes differ, first at {idx}: {[(int(a8[tuple(i)]), int(b8[tuple(i)])) for i in idx]}"


SHAPES = [(1, 128), (3, 384), (16, 7168), (127, 1664), (64, 2048), (257, 512)]


@pytest.mark.parametrize("M,K", SHAPES)
@pytest.mark.parametrize("column_major,aligned", [(False, False), (True, False), (True, True)])
def test_python_api_fp32_scales(gpu, oracle, M, K, column_major, aligned):
    """fp8_kernel.per_token_group_quant_fp8: row-major -> x * (1/s); column-major -> x / s."""
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8

    x = make_activation(M, K, zero_group_frac=0.02)
    print(f"case M={M} K={K} column_major={column_major} aligned={aligned}", flush=True)
    q, s = per_token_group_quant_fp8(x.to(gpu), 128, column_major_scales=column_major, scale_tma_aligned=aligned)
    layout = "row" if not column_major else ("col_aligned" if aligned else "col")
    q_o, s_o = oracle.group_quant(x, 128, mode="rcp" if not column_major else "div", layout=layout)
    assert q.dtype == FP8 and tuple(q.shape) == (M, K)
    assert tuple(s.shape) == tuple(s_o.shape) and s.stride() == s_o.stride()
    assert _same_bits(s, s_o)
    assert _same_bits(q, q_o), _diff_report(q, q_o)


@pytest.mark.parametrize("M,K", SHAPES)
@pytest.mark.parametrize("enable_v2", [False, True])
@pytest.mark.parametrize("layout", ["row", "col", "col_aligned", "ue8m0"])
def test_sgl_kernel_api(gpu, oracle, M, K, enable_v2, layout):
    """sglang_per_token_group_quant_fp8 -> sgl_per_token_group_quant_8bit: v1 divides, v2 multiplies by 448/amax."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8

    x = make_activation(M, K, seed=M * 7 + K, zero_group_frac=0.02)
    print(f"case M={M} K={K} v2={enable_v2} layout={layout}", flush=True)
    q, s = sglang_per_token_group_quant_fp8(
        x.to(gpu), 128, column_major_scales=layout != "row", scale_tma_aligned=layout in ("col_aligned", "ue8m0"),
        scale_ue8m0=layout == "ue8m0", enable_v2=enable_v2)
    q_o, s_o = oracle.group_quant(x, 128, mode="mul" if enable_v2 else "div", layout=layout,
                                  pow2_floor=0.0 if enable_v2 else 1e-10)
    assert tuple(s.shape) == tuple(s_o.shape) and s.stride() == s_o.stride() and s.dtype == s_o.dtype
    if layout == "ue8m0":
        G = K // 128
        assert torch.equal(oracle.unpack_ue8m0(s.cpu(), 4 * s.shape[1]), oracle.unpack_ue8m0(s_o, 4 * s.shape[1]))
        zero = x.float().view(M, G, 128).abs().amax(-1) == 0
        if zero.any():  # v1 floors the scale at 1e-10 (byte 94), v2 does not (byte 85)
            assert set(oracle.unpack_ue8m0(s.cpu(), G)[zero].tolist()) == {85 if enable_v2 else 94}
    else:
        assert _same_bits(s, s_o)
    assert _same_bits(q, q_o), _diff_report(q, q_o)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("group", [16, 32, 64, 128, 256, 512])
def test_group_sizes_and_input_dtypes(gpu, oracle, dtype, group):
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8, sglang_per_token_group_quant_8bit

    M, K = 83, 4096
    x = make_activation(M, K, seed=group, dtype=dtype, group=group, zero_group_frac=0.01)
    print(f"case dtype={dtype} group={group}", flush=True)
    q, s = per_token_group_quant_fp8(x.to(gpu), group)
    q_o, s_o = oracle.group_quant(x, group, mode="rcp")
    assert _same_bits(s, s_o) and _same_bits(q, q_o), _diff_report(q, q_o)
    q, s = sglang_per_token_group_quant_8bit(x.to(gpu), group, FP8, enable_v2=False)
    q_o, s_o = oracle.group_quant(x, group, mode="div")
    assert _same_bits(s, s_o) and _same_bits(q, q_o), _diff_report(q, q_o)
    # int8 destination: truncation toward zero, range [-128, 127]
    q, s = sglang_per_token_group_quant_8bit(x.to(gpu), group, torch.int8, enable_v2=False)
    q_o, s_o = oracle.group_quant(x, group, mode="div", dst_dtype=torch.int8)
    assert q.dtype == torch.int8 and _same_bits(s, s_o) and _same_bits(q, q_o), _diff_report(q, q_o)
    if dtype != torch.float32 and group <= 128:
        q, s = sglang_per_token_group_quant_8bit(x.to(gpu), group, torch.int8, enable_v2=True)
        q_o, s_o = oracle.group_quant(x, group, mode="mul", dst_dtype=torch.int8)
        assert _same_bits(s, s_o) and _same_bits(q, q_o), _diff_report(q, q_o)


def test_every_bf16_value_under_many_scales(gpu, oracle):
    """Brute force of the element arithmetic: each group holds its amax in slot 0 and 127 other
    bf16 values of smaller magnitude, sweeping every finite bf16 magnitude under 96 different
    scales, so a wrong rounding in the divide or in the fp8 conversion cannot hide."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8

    g = torch.Generator().manual_seed(99)
    mags = torch.arange(0x0001, 0x7F80, dtype=torch.int32)  # every positive finite bf16, subnormals included
    rows = []
    for i in range(96):
        top = int(torch.randint(0x2000, 0x7000, (1,), generator=g))  # amax between ~1e-29 and ~1e+29
        vals = mags[mags <= top]
        # pick what is closest to amax (where codes are non-zero) plus a random sample of the rest
        near = vals[-127 * 24:]
        rest = vals[torch.randperm(vals.numel(), generator=g)[: 127 * 8]]
        body = torch.cat([near, rest])
        body = body[: body.numel() // 127 * 127].view(-1, 127)
        sign = torch.randint(0, 2, body.shape, generator=g, dtype=torch.int32) << 15
        grp = torch.cat([torch.full((body.shape[0], 1), top, dtype=torch.int32), body | sign], dim=1)
        rows.append(grp)
    bits = torch.cat(rows).to(torch.int16)
    x = bits.view(torch.bfloat16).reshape(-1, 128 * 4)  # four groups per row
    for v2 in (False, True):
        q, s = sglang_per_token_group_quant_fp8(x.to(gpu), 128, enable_v2=v2)
        q_o, s_o = oracle.group_quant(x, 128, mode="mul" if v2 else "div")
        assert _same_bits(s, s_o)
        assert _same_bits(q, q_o), _diff_report(q, q_o)


def test_division_is_correctly_rounded_at_fp8_ties(gpu, oracle):
    """The divide mode computes x / s with a shared reciprocal and two FMA refinement steps.  Its quotient must be the
    correctly rounded one: fp32 inputs are placed within +-3 ulp of tie * s for every midpoint between neighbouring
    e4m3 codes, under 6000 random scales, so that a quotient wrong in its last bit lands on the other side of the tie."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_8bit

    g = torch.Generator().manual_seed(123)
    codes = torch.arange(0, 0x7E, dtype=torch.int32).to(torch.uint8)
    lo = codes.view(FP8).to(torch.float32)
    hi = (codes + 1).view(FP8).to(torch.float32)
    ties = ((lo + hi) / 2)[1:]  # 125 midpoints (skip the one next to zero: below 2^-10 everything rounds to zero)
    G = 6000
    amax = torch.exp2(torch.rand(G, generator=g) * 60 - 30) * (1 + torch.rand(G, generator=g))
    s = amax / 448.0
    x = torch.zeros(G, 128)
    x[:, 0] = amax
    t = ties[torch.randint(0, ties.numel(), (G, 127), generator=g)]
    base = t * s[:, None]
    step = torch.randint(-3, 4, (G, 127), generator=g, dtype=torch.int32)
    xi = base.view(torch.int32) + step  # move by whole ulps
    sign = torch.where(torch.rand(G, 127, generator=g) < 0.5, -1.0, 1.0)
    x[:, 1:] = xi.view(torch.float32) * sign
    x = x.reshape(G // 4, 512).contiguous()
    assert float(x.abs().view(G, 128)[:, 1:].max(dim=1).values.sub(amax).max()) <= 0  # amax really is the group maximum
    q, sc = sglang_per_token_group_quant_8bit(x.to(gpu), 128, FP8, enable_v2=False)
    q_o, s_o = oracle.group_quant(x, 128, mode="div")
    assert _same_bits(sc, s_o)
    assert _same_bits(q, q_o), _diff_report(q, q_o)
    # the construction is sharp: a reciprocal-multiply quotient does differ on this input
    q_r, _ = oracle.group_quant(x, 128, mode="rcp")
    assert int((_u8(q_r) != _u8(q_o)).sum()) > 100


def test_known_answer_construction(gpu):
    """test/srt/quant/test_fp8_kernel.py:24-100 with exactly representable scales: the quantizer must
    return the scale and the codes it was built from."""
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8

    g = torch.Generator().manual_seed(11)
    M, K, group = 256, 512, 128
    qa = torch.rand(M, K // group, group, generator=g) * 2 - 1
    qa = qa * (448.0 / qa.abs().amax(-1, keepdim=True))
    q_gt = qa.clamp(-448, 448).to(FP8)
    scale = torch.randint(1, 1 << 11, (M, K // group), generator=g).float() * torch.exp2(
        torch.randint(-20, 4, (M, K // group), generator=g).float())
    x = (q_gt.float() * scale[..., None]).view(M, K)
    for col in (False, True):
        q, s = per_token_group_quant_fp8(x.to(gpu), group, column_major_scales=col)
        assert torch.equal(s.cpu(), scale)
        assert torch.equal(_u8(q.cpu()), _u8(q_gt.view(M, K)))


def test_outliers_never_produce_nan_or_overflow(gpu):
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8

    x = make_activation(512, 4096, seed=1, outlier_frac=0.01, outlier_gain=1e4)
    x[0, :128] = 3e38  # near the bf16 maximum
    x[1, :128] = 1e-38
    for col in (False, True):
        q, s = per_token_group_quant_fp8(x.to(gpu), 128, column_major_scales=col)
        codes = _u8(q.cpu())
        assert int(((codes & 0x7F) == 0x7F).sum()) == 0  # 0x7f / 0xff are the NaN codes
        assert bool(torch.isfinite(s.cpu()).all()) and bool((s.cpu() > 0).all())


@pytest.mark.parametrize("variant", ["row_fp32", "col_ue8m0"])
def test_full_size_config(gpu, oracle, variant):
    """M=16384, K=7168 (the benchmark configuration): bit-exact against the oracle at full size, and
    the size-independent invariants (no NaN code, |q| <= 448, zero groups, amax element at +-448)."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8

    M, K = 16384, 7168
    x = make_activation(M, K, zero_group_frac=1e-4, zero_elem_frac=1e-4)
    xg = x.to(gpu)
    if variant == "row_fp32":
        q, s = sglang_per_token_group_quant_fp8(xg, 128, enable_v2=False)
        q_o, s_o = oracle.group_quant(x, 128, mode="div", layout="row")
        assert _same_bits(s, s_o)
    else:
        q, s = sglang_per_token_group_quant_fp8(xg, 128, column_major_scales=True, scale_tma_aligned=True,
                                                scale_ue8m0=True, enable_v2=True)
        q_o, s_o = oracle.group_quant(x, 128, mode="mul", layout="ue8m0")
        assert s.stride() == (1, M) and tuple(s.shape) == (M, 14)
        assert torch.equal(oracle.unpack_ue8m0(s.cpu(), 56), oracle.unpack_ue8m0(s_o, 56))
    assert _same_bits(q, q_o), _diff_report(q, q_o)
    codes = _u8(q.cpu())
    assert int(((codes & 0x7F) == 0x7F).sum()) == 0
    xf = x.float().view(M, K // 128, 128)
    zero = xf.abs().amax(-1) == 0
    assert zero.any() and bool((codes.view(M, K // 128, 128)[zero] == 0).all())
    if variant == "row_fp32":
        top = q.cpu().float().view(M, K // 128, 128).gather(-1, xf.abs().argmax(-1, keepdim=True)).squeeze(-1).abs()
        assert bool((top[~zero] == 448).all())


def test_runs_on_the_current_stream_and_leaves_neighbours_alone(gpu):
    """The kernel must honour the caller's stream and write nothing outside its outputs."""
    from sglang_amd.fp8_kernel import create_per_token_group_quant_fp8_output_scale
    from sglang_amd.sgl_kernel import sgl_per_token_group_quant_fp8

    M, K = 37, 640
    x = make_activation(M, K, seed=5).to(gpu)
    pad = 256
    qbuf = torch.full((M * K + 2 * pad,), 0xAB, dtype=torch.uint8, device=gpu)
    q = qbuf[pad : pad + M * K].view(M, K).view(FP8)
    s = create_per_token_group_quant_fp8_output_scale((M, K), gpu, 128, False, False, False)
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        sgl_per_token_group_quant_fp8(x, q, s, 128, 1e-10, -448.0, 448.0)
    st.synchronize()
    assert bool((qbuf[:pad] == 0xAB).all()) and bool((qbuf[-pad:] == 0xAB).all())
    assert bool((s > 0).all())
