"""Pins the oracle's number-format conversions against torch's CPU routines (a library
implementation the oracle shares no code with), exhaustively where the domain is small."""
import torch


def _all_bf16_as_f32():
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    return bits.view(torch.bfloat16).to(torch.float32)


def _all_f16_as_f32():
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    return bits.view(torch.float16).to(torch.float32)


def _finite_mask(x):
    return torch.isfinite(x)


def test_e4m3fn_decode_all_codes(oracle):
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    want = codes.view(torch.float8_e4m3fn).to(torch.float32)
    got = oracle.e4m3fn_decode(codes)
    nan = torch.isnan(want)
    assert nan.sum() == 2 and torch.equal(torch.isnan(got), nan)
    assert torch.equal(got[~nan].view(torch.int32), want[~nan].view(torch.int32))  # bitwise, keeps -0


def test_e4m3fn_encode_every_bf16_and_f16_value(oracle):
    for x in (_all_bf16_as_f32(), _all_f16_as_f32()):
        x = x[_finite_mask(x)]
        want = x.to(torch.float8_e4m3fn).view(torch.uint8)
        got = oracle.e4m3fn_encode(x)
        assert torch.equal(got, want)


def test_e4m3fn_encode_random_fp32_and_ties(oracle):
    g = torch.Generator().manual_seed(1)
    # log-uniform magnitudes across the whole fp8 range and beyond, both signs
    mag = torch.exp2(torch.rand(2_000_000, generator=g) * 24 - 14)
    sign = torch.where(torch.rand(2_000_000, generator=g) < 0.5, -1.0, 1.0)
    x = mag * sign
    assert torch.equal(oracle.e4m3fn_encode(x), x.to(torch.float8_e4m3fn).view(torch.uint8))
    # exact midpoints between neighbouring codes (ties must go to the even code), and 1 ulp either side
    codes = torch.arange(0, 0x7E, dtype=torch.int32).to(torch.uint8)
    lo = codes.view(torch.float8_e4m3fn).to(torch.float32)
    hi = (codes + 1).view(torch.float8_e4m3fn).to(torch.float32)
    mid = (lo + hi) / 2
    pts = torch.cat([mid, torch.nextafter(mid, hi), torch.nextafter(mid, lo)])
    pts = torch.cat([pts, -pts, torch.tensor([0.0, -0.0, 448.0, -448.0, 463.9, 464.0, 2.0**-10, 2.0**-10 * 1.0001])])
    assert torch.equal(oracle.e4m3fn_encode(pts), pts.to(torch.float8_e4m3fn).view(torch.uint8))
    # scalar entry point agrees with the batch one
    L = oracle.lib()
    for v in (0.3, -0.0019, 448.0, 1e-3, 17.0):
        assert L.oracle_e4m3fn_encode(v) == int(torch.tensor(v).to(torch.float8_e4m3fn).view(torch.uint8))
    assert L.oracle_e4m3fn_encode(0.3) == 0x2A and L.oracle_e4m3fn_encode(-0.0019) == 0x81


def test_e4m3fn_out_of_range_is_nan_not_saturated(oracle):
    x = torch.tensor([480.0, 500.0, -1e9, float("inf"), float("nan")])
    got = oracle.e4m3fn_encode(x)
    assert [int(v) & 0x7F for v in got] == [0x7F] * 5
    assert torch.equal(got[:3], x[:3].to(torch.float8_e4m3fn).view(torch.uint8))


def test_f32_to_bf16_and_f16(oracle):
    g = torch.Generator().manual_seed(2)
    mag = torch.exp2(torch.rand(1_000_000, generator=g) * 60 - 30)
    x = mag * torch.where(torch.rand(1_000_000, generator=g) < 0.5, -1.0, 1.0)
    edge = torch.tensor([0.0, -0.0, 65504.0, 65519.9, 65520.0, 65536.0, 1e38, 3.3e38, 2.0**-24, 2.0**-25,
                         2.0**-25 * 1.0001, 6e-8, 5.96e-8, 6.1e-5, 6.0e-5, float("inf"), -float("inf")])
    x = torch.cat([x, edge, _all_f16_as_f32()[_finite_mask(_all_f16_as_f32())]])
    assert torch.equal(oracle.f32_to_bf16_bits(x), x.to(torch.bfloat16).view(torch.int16))
    assert torch.equal(oracle.f32_to_f16_bits(x), x.to(torch.float16).view(torch.int16))
    # ties of bf16: low half exactly 0x8000
    base = torch.randint(0, 0x7F00, (100000,), generator=g, dtype=torch.int32)
    tie = ((base << 16) | 0x8000).view(torch.float32)
    assert torch.equal(oracle.f32_to_bf16_bits(tie), tie.to(torch.bfloat16).view(torch.int16))


def test_f16_to_f32_all_codes(oracle):
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    want = bits.view(torch.float16).to(torch.float32)
    got = oracle.f16_bits_to_f32(bits)
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan)
    assert torch.equal(got[~nan].view(torch.int32), want[~nan].view(torch.int32))
