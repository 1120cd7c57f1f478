"""Pins the oracle's group quantizer.

Checks are chosen so that a plausible slip (wrong rounding mode, eps applied in the input
dtype, a scale written to the wrong slot, an off-by-one exponent) fails at least one:
  * torch's own CPU fp32 divide / multiply / float8 cast as an independent routine,
    arranged like the reference's torch-native test helper
    (python/sglang/test/test_block_fp8.py:23-48);
  * the known-answer construction of test/srt/quant/test_fp8_kernel.py:24-45;
  * closed forms and invariants (|q| <= 448, the amax element maps to +-448, zero groups);
  * power-of-two scales: fp64 ceil(log2), exact powers of two and their 1-ulp neighbours;
  * layout algebra: every layout unpacks to the same row-major scales, padding is zero.
"""
import math

import pytest
import torch

from sglang_amd.workloads import make_activation

FP8 = torch.float8_e4m3fn


def _torch_group_quant(x, group, mode):
    """fp32 torch restatement; eps clamp done in fp32 (both real kernels do that)."""
    M, K = x.shape
    xf = x.to(torch.float32).view(M, K // group, group)
    amax = xf.abs().amax(-1, keepdim=True).clamp(min=1e-10)
    if mode == "div":
        s = amax / 448.0
        t = xf / s
    elif mode == "rcp":
        s = amax / 448.0
        t = xf * (1.0 / s)
    else:
        s = amax * torch.tensor(1.0 / 448.0, dtype=torch.float32)
        t = xf * (torch.full_like(amax, 448.0) / amax)  # true division; `448.0 / t` is reciprocal()*448 in torch
    q = t.clamp(-448.0, 448.0).to(FP8).view(M, K)
    return q, s.view(M, K // group)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("mode", ["div", "rcp", "mul"])
@pytest.mark.parametrize("group", [16, 64, 128, 256])
def test_matches_torch_fp32_arithmetic(oracle, dtype, mode, group):
    x = make_activation(37, 1024, seed=group + 7, dtype=dtype, zero_group_frac=0.02, group=group)
    q, s = oracle.group_quant(x, group, mode=mode)
    q_t, s_t = _torch_group_quant(x, group, mode)
    assert torch.equal(s.view(torch.int32), s_t.view(torch.int32))
    assert torch.equal(q.view(torch.uint8), q_t.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mode", ["div", "rcp"])
@pytest.mark.parametrize("K", [1536, 7168])
def test_whole_row_groups_match_torch_fp32_arithmetic(oracle, dtype, mode, K):
    """group == K (a weight quantized per output channel at load time): the same routine over one long group."""
    x = make_activation(9, K, seed=K + 3, dtype=dtype)
    x[2] = 0
    q, s = oracle.group_quant(x, K, mode=mode)
    q_t, s_t = _torch_group_quant(x, K, mode)
    assert tuple(s.shape) == (9, 1)
    assert torch.equal(s.view(torch.int32), s_t.view(torch.int32))
    assert torch.equal(q.view(torch.uint8), q_t.view(torch.uint8))


def test_modes_differ_somewhere_but_only_by_one_code(oracle):
    # guards against the three modes being wired to the same arithmetic
    x = make_activation(256, 2048, seed=3)
    q = {m: oracle.group_quant(x, 128, mode=m)[0].view(torch.uint8).to(torch.int16) for m in ("div", "rcp", "mul")}
    for a, b in (("div", "rcp"), ("div", "mul")):
        d = (q[a] - q[b]).abs()
        assert 0 < int((d != 0).sum()) < 0.005 * d.numel()
        assert int(d.max()) == 1


def _known_answer(M, K, group, seed):
    """q_gt on the fp8 grid with |max| = 448 per group; scale with a short mantissa so that
    q_gt * scale, 448 * scale and (448 * scale) / 448 are all exact in fp32."""
    g = torch.Generator().manual_seed(seed)
    qa = torch.rand(M, K // group, group, generator=g) * 2 - 1
    qa = qa * (448.0 / qa.abs().amax(-1, keepdim=True))
    q_gt = qa.clamp(-448, 448).to(FP8)
    # make sure each group really contains +-448
    assert bool((q_gt.to(torch.float32).abs().amax(-1) == 448).all())
    mant = torch.randint(1, 1 << 11, (M, K // group), generator=g).to(torch.float32)
    expo = torch.randint(-20, 4, (M, K // group), generator=g).to(torch.float32)
    scale = mant * torch.exp2(expo)
    x = (q_gt.to(torch.float32) * scale[..., None]).view(M, K)
    return x, q_gt.view(M, K), scale


@pytest.mark.parametrize("mode", ["div", "rcp", "mul"])
def test_known_answer_construction(oracle, mode):
    x, q_gt, scale = _known_answer(64, 512, 128, seed=11)
    q, s = oracle.group_quant(x, 128, mode=mode)
    if mode == "mul":  # amax * (1/448f) is rounded twice; the reference's own test allows 1.3e-6 relative
        torch.testing.assert_close(s, scale)
    else:
        assert torch.equal(s, scale)
    assert torch.equal(q.view(torch.uint8), q_gt.view(torch.uint8))


def test_invariants_and_zero_groups(oracle):
    x = make_activation(128, 1024, seed=5, zero_group_frac=0.05)
    xf = x.to(torch.float32).view(128, 8, 128)
    zero = xf.abs().amax(-1) == 0
    assert zero.any()
    for mode in ("div", "rcp", "mul"):
        q, s = oracle.group_quant(x, 128, mode=mode)
        qf = q.to(torch.float32).view(128, 8, 128)
        assert not torch.isnan(qf).any() and float(qf.abs().max()) <= 448.0
        # zero groups: q == 0 and the scale is eps/448 (mode mul: eps * (1/448))
        assert bool((qf[zero] == 0).all())
        want = (torch.tensor(1e-10) / 448.0) if mode != "mul" else torch.tensor(1e-10) * torch.tensor(1.0 / 448.0)
        assert bool((s[zero] == want).all())
        # scale closed form on the other groups
        amax = xf.abs().amax(-1)
        want_s = amax / 448.0 if mode != "mul" else amax * torch.tensor(1.0 / 448.0)
        assert torch.equal(s[~zero], want_s[~zero])
    # in DIV mode the element that attains amax is exactly +-448
    q, _ = oracle.group_quant(x, 128, mode="div")
    qf = q.to(torch.float32).view(128, 8, 128)
    idx = xf.abs().argmax(-1, keepdim=True)
    top = qf.gather(-1, idx).squeeze(-1).abs()
    assert bool((top[~zero] == 448).all())


def test_eps_is_applied_in_fp32_not_in_the_input_dtype(oracle):
    # bf16(1e-10) != 1e-10f; a group whose amax is below eps must give exactly 1e-10f/448
    x = torch.full((1, 128), 3e-11, dtype=torch.bfloat16)
    _, s = oracle.group_quant(x, 128, mode="div")
    assert float(s[0, 0]) == float(torch.tensor(1e-10) / 448.0)


def test_int8_destination_truncates(oracle):
    x = make_activation(32, 512, seed=9)
    q, s = oracle.group_quant(x, 128, mode="div", dst_dtype=torch.int8)
    xf = x.to(torch.float32).view(32, 4, 128)
    amax = xf.abs().amax(-1, keepdim=True).clamp(min=1e-10)
    s_t = amax / 127.0
    q_t = (xf / s_t).clamp(-128, 127).to(torch.int8).view(32, 512)  # torch's float->int8 cast truncates toward zero
    assert torch.equal(s, s_t.view(32, 4)) and torch.equal(q, q_t)
    frac = (xf / s_t).view(32, 512)
    assert bool((q.to(torch.float32).abs() <= frac.abs()).all())  # never rounds away from zero


# ---------------------------------------------------------------- power-of-two scales

def _positive_normal_bf16():
    bits = torch.arange(0x0080, 0x7F80, dtype=torch.int32).to(torch.int16)
    return bits.view(torch.bfloat16)


def test_ue8m0_exponent_for_every_positive_normal_bf16_amax(oracle):
    amax = _positive_normal_bf16()
    amax = amax[amax.to(torch.float32) >= 1e-10]  # below eps the group behaves like a zero group
    M = amax.numel()
    x = torch.zeros(M, 128, dtype=torch.bfloat16)
    x[:, 5] = amax
    want = torch.ceil(torch.log2(amax.to(torch.float64) / 448.0)).to(torch.int64) + 127
    for mode in ("mul", "div", "rcp"):
        _, s = oracle.group_quant(x, 128, mode=mode, layout="ue8m0")
        got = oracle.unpack_ue8m0(s, 1).view(-1).to(torch.int64)
        assert torch.equal(got, want), mode


def test_ue8m0_powers_of_two_and_neighbours(oracle):
    # amax = 448 * 2^k (fp32 input so that 1-ulp neighbours exist) -> exactly 2^k; one ulp above -> 2^(k+1)
    ks = torch.arange(-30, 30)
    amax = 448.0 * torch.exp2(ks.to(torch.float32))
    up = torch.nextafter(amax, torch.tensor(float("inf")))
    dn = torch.nextafter(amax, torch.tensor(0.0))
    for vals, want in ((amax, ks + 127), (up, ks + 128), (dn, ks + 127)):
        x = torch.zeros(len(ks), 128, dtype=torch.float32)
        x[:, 0] = -vals
        for mode in ("div", "mul"):
            _, s = oracle.group_quant(x, 128, mode=mode, layout="ue8m0")
            got = oracle.unpack_ue8m0(s, 1).view(-1).to(torch.int64)
            if mode == "mul" and vals is dn:
                # amax*(1/448f) rounds; the reference's v2 kernel has the same property, so only bound it
                assert bool(((got - want).abs() <= 1).all())
            else:
                assert torch.equal(got, want), (mode,)


def test_ue8m0_zero_group_bytes(oracle):
    x = torch.zeros(4, 512, dtype=torch.bfloat16)
    _, s = oracle.group_quant(x, 128, mode="mul", layout="ue8m0")
    assert set(oracle.unpack_ue8m0(s, 4).view(-1).tolist()) == {85}  # 1e-10/448 = 2^-42.03 -> 2^-42
    _, s = oracle.group_quant(x, 128, mode="div", layout="ue8m0", pow2_floor=1e-10)
    assert set(oracle.unpack_ue8m0(s, 4).view(-1).tolist()) == {94}  # ceil(log2(1e-10)) = -33
    assert math.ceil(math.log2(1e-10 / 448)) + 127 == 85 and math.ceil(math.log2(1e-10)) + 127 == 94


def test_pow2_scales_make_all_modes_identical(oracle):
    x = make_activation(64, 1024, seed=21, zero_group_frac=0.05)
    outs = [oracle.group_quant(x, 128, mode=m, layout="ue8m0") for m in ("div", "rcp", "mul")]
    for q, s in outs[1:]:
        assert torch.equal(q.view(torch.uint8), outs[0][0].view(torch.uint8))
        assert torch.equal(s, outs[0][1])
    # and q equals x / 2^e computed independently
    e = oracle.unpack_ue8m0(outs[0][1], 8).to(torch.float32) - 127
    t = (x.to(torch.float32).view(64, 8, 128) / torch.exp2(e)[..., None]).clamp(-448, 448)
    assert torch.equal(outs[0][0].view(torch.uint8), t.to(FP8).view(64, 1024).view(torch.uint8))


# ---------------------------------------------------------------- scale layouts

@pytest.mark.parametrize("M,K", [(1, 128), (5, 640), (16, 7168), (127, 384), (130, 1664)])
def test_layouts_hold_the_same_scales(oracle, M, K):
    x = make_activation(M, K, seed=M + K)
    q0, s_row = oracle.group_quant(x, 128, mode="div", layout="row")
    assert s_row.is_contiguous() and tuple(s_row.shape) == (M, K // 128)
    for layout in ("col", "col_aligned"):
        q, s = oracle.group_quant(x, 128, mode="div", layout=layout)
        assert tuple(s.shape) == (M, K // 128)
        assert s.stride(0) == 1 and s.stride(1) == (M if layout == "col" else (M + 3) // 4 * 4)
        assert torch.equal(s, s_row) and torch.equal(q.view(torch.uint8), q0.view(torch.uint8))


@pytest.mark.parametrize("M,K", [(1, 128), (5, 640), (16, 7168), (127, 384), (130, 1664)])
def test_packed_layout_algebra(oracle, M, K):
    G = K // 128
    x = make_activation(M, K, seed=M * 3 + K)
    _, s = oracle.group_quant(x, 128, mode="mul", layout="ue8m0")
    assert s.dtype == torch.int32 and tuple(s.shape) == (M, (G + 3) // 4)
    assert s.stride(0) == 1 and s.stride(1) == (M + 3) // 4 * 4
    # bytes -> exponents -> the same power-of-two scales as the unpacked computation
    xf = x.to(torch.float32).view(M, G, 128)
    t = xf.abs().amax(-1).clamp(min=1e-10) * torch.tensor(1.0 / 448.0)
    want = torch.ceil(torch.log2(t.to(torch.float64))).to(torch.int64) + 127
    assert torch.equal(oracle.unpack_ue8m0(s, G).to(torch.int64), want)
    by = oracle.unpack_ue8m0(s, 4 * s.shape[1])
    assert bool((by[:, G:] == 0).all())  # padding bytes of the last word are zero
    # word w of row m sits at element offset w * align4(M) + m of the underlying storage
    base = s.as_strided((s.stride(1) * s.shape[1],), (1,))
    for m in (0, M - 1):
        for w in (0, s.shape[1] - 1):
            assert int(base[w * s.stride(1) + m]) == int(s[m, w])


def test_per_token_quant_int8(oracle):
    x = make_activation(64, 4096, seed=31)
    q, s = oracle.per_token_quant_int8(x)
    xf = x.to(torch.float32)
    amax = xf.abs().amax(1, keepdim=True).clamp(min=1e-10)
    t = xf * (torch.full_like(amax, 127.0) / amax)
    want = (torch.sign(t) * torch.floor(t.abs() + 0.5)).to(torch.int8)  # round half away from zero
    assert torch.equal(q, want) and torch.equal(s, amax / 127.0)
    assert int(q.abs().max()) == 127


# ---------------------------------------------------------------- per-token FP8 quantizer (one scale per row)

@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_per_token_quant_fp8_against_torch_fp32(oracle, dtype):
    """sgl-kernel/csrc/gemm/per_token_quant_fp8.cu:15-85 restated with torch CPU fp32 ops (IEEE `/` and `*`) and torch's
    own e4m3fn cast: scale = amax / 448, q = clamp(x * (1 / scale)), zero rows -> scale 0, codes 0."""
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(37, 1024, generator=g) * torch.rand(37, 1, generator=g) * 20).to(dtype)
    x[5] = 0
    x[6, 17] = 3.0e4 if dtype != torch.float16 else 6.0e4  # an outlier that sets the row's scale
    q, s = oracle.per_token_quant_fp8(x)
    xf = x.float()
    s_ref = xf.abs().amax(dim=1, keepdim=True) / 448.0
    inv = torch.where(s_ref == 0, torch.zeros(()), 1.0 / s_ref)
    q_ref = (xf * inv).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    assert torch.equal(s.view(torch.int32), s_ref.view(torch.int32))
    assert torch.equal(q.view(torch.uint8), q_ref.view(torch.uint8))
    assert float(s[5]) == 0.0 and not bool(q[5].view(torch.uint8).any())
    # the element that attains the row maximum encodes to +-448 (0x7e / 0xfe)
    assert int(q[6, 17].view(torch.uint8)) == 0x7E


def test_per_token_quant_fp8_known_answer(oracle):
    """Codes that are exactly representable times a power-of-two scale must come back unchanged, with that scale."""
    g = torch.Generator().manual_seed(4)
    codes = torch.randint(0, 256, (16, 256), generator=g, dtype=torch.uint8)
    codes = torch.where((codes & 0x7F) == 0x7F, codes & 0xF7, codes)
    codes[:, 0] = 0x7E  # every row attains 448
    scale = torch.exp2(torch.randint(-6, 7, (16, 1), generator=g).float())
    x = codes.view(torch.float8_e4m3fn).float() * scale
    q, s = oracle.per_token_quant_fp8(x)
    assert torch.equal(s, scale)
    back = q.view(torch.uint8)
    want = torch.where(codes == 0x80, torch.zeros((), dtype=torch.uint8), codes)  # -0 * scale = -0 -> encodes as 0x80 again
    assert torch.equal(back, codes) or torch.equal(back, want)


# ---------------------------------------------------------------- per-tensor FP8 quantizer (one scale for the tensor)

@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_per_tensor_quant_fp8_against_torch_fp32(oracle, dtype):
    """sgl-kernel/csrc/gemm/per_tensor_quant_fp8.cu:10-100 restated with torch CPU fp32 ops and torch's e4m3fn cast:
    scale = amax / 448 (dynamic) or given (static), q = clamp(x * (1 / scale))."""
    g = torch.Generator().manual_seed(11)
    x = (torch.randn(29, 1000, generator=g) * 7).to(dtype)  # 29000 elements: not a multiple of a 16-byte vector
    x[3, 7] = -2.5e4
    q, s = oracle.per_tensor_quant_fp8(x)
    xf = x.float()
    s_ref = (xf.abs().max() / 448.0).reshape(1)
    q_ref = (xf * (1.0 / s_ref)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    assert torch.equal(s.view(torch.int32), s_ref.view(torch.int32))
    assert torch.equal(q.view(torch.uint8), q_ref.view(torch.uint8))
    assert int(q[3, 7].view(torch.uint8)) == 0xFE  # the extreme element encodes to -448
    # static: a scale that saturates part of the tensor and is not a power of two
    given = torch.tensor([0.013], dtype=torch.float32)
    q2, s2 = oracle.per_tensor_quant_fp8(x, given)
    q2_ref = (xf * (1.0 / given)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    assert torch.equal(s2, given) and torch.equal(q2.view(torch.uint8), q2_ref.view(torch.uint8))
    assert int((q2.view(torch.uint8) & 0x7F).max()) == 0x7E  # saturated, never NaN


def test_per_tensor_quant_fp8_known_answer_and_zero_tensor(oracle):
    """Representable codes times a power-of-two scale come back unchanged with that scale; a tensor of zeros gets
    scale 0 and, because fmin/fmax drop the NaN of 0 * inf, codes of +448 (what the reference's kernel produces)."""
    g = torch.Generator().manual_seed(12)
    codes = torch.randint(0, 256, (8, 512), generator=g, dtype=torch.uint8)
    codes = torch.where((codes & 0x7F) == 0x7F, codes & 0xF7, codes)
    codes[0, 0] = 0x7E
    x = codes.view(torch.float8_e4m3fn).float() * 0.25
    q, s = oracle.per_tensor_quant_fp8(x)
    assert float(s) == 0.25
    assert torch.equal(q.view(torch.uint8), codes)
    qz, sz = oracle.per_tensor_quant_fp8(torch.zeros(4, 64))
    assert float(sz) == 0.0 and bool((qz.view(torch.uint8) == 0x7E).all())


# ---------------------------------------------------------------- silu(gate) * up in front of the v2 quantizer

def test_oracle_expf_within_one_ulp(oracle):
    """The oracle's exp is built from individually rounded fp32 operations (so that the GPU kernel can repeat it bit for
    bit); against fp64 exp it must stay within 1 ulp over the whole range, with exact limits."""
    import math

    g = torch.Generator().manual_seed(21)
    xs = torch.cat([torch.linspace(-104.0, 88.7, 20001), torch.randn(20000, generator=g) * 4, torch.tensor([0.0, -0.0, 1.0, -1.0])])
    worst = 0.0
    for v in xs.tolist():
        got = oracle.expf(v)
        want = math.exp(v)
        want32 = float(torch.tensor(want, dtype=torch.float64).to(torch.float32))
        if want32 == 0.0 or math.isinf(want32) or want < 1.2e-38:
            continue  # subnormal results only need to vanish next to 1
        ulp = abs(float(torch.nextafter(torch.tensor(want32), torch.tensor(float("inf")))) - want32)
        worst = max(worst, abs(got - want) / ulp)
    assert worst <= 1.0, worst
    assert oracle.expf(0.0) == 1.0 and oracle.expf(100.0) == float("inf") and oracle.expf(-200.0) == 0.0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_silu_mul_against_torch(oracle, dtype):
    """per_token_group_quant_8bit_v2.cu:318-331: T(silu(float(gate))) * up in T.  torch's CPU silu uses a correctly
    rounded-ish exp, the oracle its own 1-ulp exp, so after rounding to T the two may differ in isolated elements by one
    unit of T; a wrong formula (activation not rounded to T first, halves swapped, product in fp32) differs everywhere."""
    g = torch.Generator().manual_seed(22)
    x = (torch.randn(64, 2 * 1024, generator=g) * 3).to(dtype)
    x[0, :8] = torch.tensor([0.0, -0.0, 30.0, -30.0, 100.0, -100.0, 1e-3, -1e-3]).to(dtype)
    got = oracle.silu_mul(x)
    gate, up = x[:, :1024], x[:, 1024:]
    want = torch.nn.functional.silu(gate.float()).to(dtype) * up
    assert got.shape == want.shape and got.dtype == dtype
    diff = (got.view(torch.int16).int() - want.view(torch.int16).int()).abs()
    assert int(diff.max()) <= 1 and float((diff != 0).float().mean()) < 2e-4, (int(diff.max()), float((diff != 0).float().mean()))
    # discriminating alternatives must be far away
    alt = (torch.nn.functional.silu(gate.float()) * up.float()).to(dtype)  # product before the first rounding
    assert float((alt.view(torch.int16) != got.view(torch.int16)).float().mean()) > 0.05


# ---------------------------------------------------------------- weight side: 128 x 128 block cast / dequant

def _ref_per_block_cast_to_fp8(x):
    """per_block_cast_to_fp8 + ceil_to_ue8m0 of python/sglang/srt/layers/quantization/fp8_utils.py:487-505, in the same
    torch operations (CPU)."""
    m, n = x.shape
    pm, pn = (m + 127) // 128 * 128, (n + 127) // 128 * 128
    x_padded = torch.zeros((pm, pn), dtype=x.dtype)
    x_padded[:m, :n] = x
    x_view = x_padded.view(-1, 128, pn // 128, 128)
    x_amax = x_view.abs().float().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
    sf = torch.pow(2.0, torch.ceil(torch.log2((x_amax / 448.0).abs())))
    x_scaled = (x_view * (1.0 / sf)).to(torch.float8_e4m3fn)
    return x_scaled.view_as(x_padded)[:m, :n].contiguous(), sf.view(x_view.size(0), x_view.size(2))


@pytest.mark.parametrize("shape", [(256, 384), (130, 200), (128, 128), (5, 7), (384, 1000)])
def test_block_cast_to_fp8_against_torch(oracle, shape):
    g = torch.Generator().manual_seed(shape[0] * 7 + shape[1])
    x = (torch.randn(*shape, generator=g) * torch.rand(*shape, generator=g).pow(4) * 3).to(torch.bfloat16)
    x[0, 0] = 448.0 * 0.25  # amax / 448 exactly a power of two in the first block: ceil must not step up
    q, s = oracle.block_cast_to_fp8(x)
    q_ref, s_ref = _ref_per_block_cast_to_fp8(x)
    assert torch.equal(s, s_ref)
    assert torch.equal(q.view(torch.uint8), q_ref.view(torch.uint8))
    assert float(s[0, 0]) == 0.25 or shape == (5, 7) and float(s[0, 0]) == 0.25
    assert bool(((q.view(torch.uint8) & 0x7F) <= 0x7E).all())  # never NaN: |x / s| <= 448
    z, sz = oracle.block_cast_to_fp8(torch.zeros(130, 130, dtype=torch.bfloat16))
    assert not bool(z.view(torch.uint8).any()) and bool((sz == 2.0 ** -22).all())  # floor 1e-4 / 448 rounds up to 2^-22


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_block_dequant_against_torch(oracle, dtype):
    g = torch.Generator().manual_seed(31)
    n, k = 200, 300
    codes = torch.randint(0, 256, (n, k), generator=g, dtype=torch.uint8)
    codes = torch.where((codes & 0x7F) == 0x7F, codes & 0xF7, codes)
    q = codes.view(torch.float8_e4m3fn)
    s = torch.rand(2, 3, generator=g) * 0.01 + 1e-4
    out = oracle.block_dequant_fp8(q, s, dtype)
    ref = (q.to(torch.float32) * s.repeat_interleave(128, 0).repeat_interleave(128, 1)[:n, :k]).to(dtype)
    assert torch.equal(out.view(torch.int16 if dtype != torch.float32 else torch.int32),
                       ref.view(torch.int16 if dtype != torch.float32 else torch.int32))


def test_row_sum_known_answers(oracle):
    """per_token_row_sum against sums that can be written down: small integers (exact in every type), a row whose terms
    cancel to one survivor, and Python's exactly rounded fsum on random fp32 rows."""
    import math

    x = torch.tensor([[1.0, 2.0, 3.0, -4.0], [0.5, 0.25, -0.75, 100.0]], dtype=torch.bfloat16)
    exact, mag, rounded = oracle.per_token_row_sum(x)
    assert exact.tolist() == [2.0, 100.0] and mag.tolist() == [10.0, 101.5] and rounded.dtype == torch.bfloat16
    assert rounded.tolist() == [2.0, 100.0]
    y = torch.randn(3, 1000, generator=torch.Generator().manual_seed(0))
    exact, mag, rounded = oracle.per_token_row_sum(y)
    for r in range(3):
        assert abs(float(exact[r]) - math.fsum(y[r].double().tolist())) <= 1e-12 * float(mag[r])
        assert float(rounded[r]) == float(torch.tensor(math.fsum(y[r].double().tolist())).float())
