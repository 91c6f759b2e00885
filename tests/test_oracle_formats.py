"""The oracle's hand-written number-format conversions against torch's casts (library routines)."""

import torch

from oracle import c_oracle as C
from tests.exact_arith import Fraction, e4m3_code, rn_e4m3


def test_f32_to_e4m3fn_dense_sweep():
    # every fp32 whose low 8 mantissa bits are zero: 2^24 patterns, covers all exponents, all rounding
    # boundaries of a 3-bit mantissa, subnormal results, overflow to NaN, Inf and NaN
    bits = (torch.arange(0, 2 ** 24, dtype=torch.int64) << 8).to(torch.int32)
    x = bits.view(torch.float32)
    want = x.to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(C.f32_to_e4m3fn(x), want)


def test_f32_to_e4m3fn_around_every_boundary():
    # all representable magnitudes, the midpoints between neighbours, and one fp32 ulp either side
    codes = torch.arange(0, 0x7F, dtype=torch.int32).to(torch.uint8)
    vals = codes.view(torch.float8_e4m3fn).to(torch.float32)
    mids = (vals[:-1] + vals[1:]) / 2
    pts = torch.cat([vals, mids, torch.tensor([464.0, 480.0, 2.0 ** -10, 2.0 ** -11])])
    b = pts.view(torch.int32)
    pts = torch.cat([pts, (b + 1).view(torch.float32), (b - 1).clamp(min=0).view(torch.float32)])
    pts = torch.cat([pts, -pts])
    want = pts.to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(C.f32_to_e4m3fn(pts), want)


def test_f32_to_e4m3fn_known_answers():
    # values worked out by hand from the format definition
    x = torch.tensor([448.0, 464.0, 464.1, 2.0 ** -10, 1.5 * 2.0 ** -9, 2.5 * 2.0 ** -9, 17.0, 19.0, -0.0, 0.0,
                      float("inf"), -float("inf"), 1e9, -448.0, 2.0 ** -6, 0.875 * 2.0 ** -6])
    want = [0x7E, 0x7E, 0x7F, 0x00, 0x02, 0x02, 0x58, 0x5A, 0x80, 0x00, 0x7F, 0xFF, 0x7F, 0xFE, 0x08, 0x07]
    assert C.f32_to_e4m3fn(x).tolist() == want
    nan = C.f32_to_e4m3fn(torch.tensor([float("nan")]))
    assert nan.item() & 0x7F == 0x7F


def test_f32_to_e4m3fn_exact_rational():
    # independent derivation: exact rational rounding to 4 significant bits, then encode
    g = torch.Generator().manual_seed(5)
    x = (torch.rand(4000, generator=g) * 2 - 1) * 448
    x = torch.cat([x, x * 2.0 ** -7, x * 2.0 ** -12])
    got = C.f32_to_e4m3fn(x).tolist()
    for v, c in zip(x.tolist(), got):
        fr = Fraction(v)
        assert c == e4m3_code(rn_e4m3(fr), negative_zero=(v < 0)), v


def test_e4m3fn_to_f32_all_codes():
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    want = codes.view(torch.float8_e4m3fn).to(torch.float32)
    got = C.e4m3fn_to_f32(codes)
    finite = ~want.isnan()
    assert torch.equal(got.isnan(), want.isnan())
    assert torch.equal(got[finite].view(torch.int32), want[finite].view(torch.int32))
    assert codes[want.isnan()].tolist() == [0x7F, 0xFF]


def test_f32_to_bf16_sweep():
    g = torch.Generator().manual_seed(1)
    bits = torch.randint(-2 ** 31, 2 ** 31 - 1, (1 << 22,), generator=g, dtype=torch.int64).to(torch.int32)
    # plus every tie pattern (low half exactly 0x8000) for a spread of high halves
    hi = torch.arange(0, 65536, dtype=torch.int64)
    ties = ((hi << 16) | 0x8000).to(torch.int32)
    x = torch.cat([bits, ties]).view(torch.float32)
    x = x[~x.isnan()]
    want = x.to(torch.bfloat16).view(torch.int16)
    assert torch.equal(C.f32_to_bf16(x).view(torch.int16), want)


def test_f32_to_f16_sweep_and_every_boundary():
    g = torch.Generator().manual_seed(2)
    bits = torch.randint(-2 ** 31, 2 ** 31 - 1, (1 << 22,), generator=g, dtype=torch.int64).to(torch.int32)
    # every finite fp16 value, the midpoint to its upper neighbour, and one fp32 ulp either side of both:
    # all rounding boundaries, the subnormal range, the step to infinity at 65520
    h = torch.arange(0, 0x7C00, dtype=torch.int32).to(torch.int16).view(torch.float16).to(torch.float32)
    nxt = torch.cat([h[1:], torch.tensor([65536.0])])
    pts = torch.cat([h, (h + nxt) / 2, torch.tensor([2.0 ** -25, 2.0 ** -26, 65519.99, 65520.0, 1e30, float("inf")])])
    b = pts.view(torch.int32)
    pts = torch.cat([pts, (b + 1).view(torch.float32), (b - 1).clamp(min=0).view(torch.float32)])
    x = torch.cat([bits.view(torch.float32), pts, -pts])
    x = x[~x.isnan()]
    assert torch.equal(C.f32_to_f16(x).view(torch.int16), x.to(torch.float16).view(torch.int16))
    assert C.f32_to_f16(torch.tensor([float("nan")])).isnan().all()
