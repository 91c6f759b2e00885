"""Pins the FP8 part of the oracle: scalar C restatement vs op-for-op torch restatement, hand-derived
known answers, exact rational arithmetic on tiny inputs, and the invariants / known-answer tests the
reference's own test-suite holds for this path."""

import pytest
import torch

from oracle import c_oracle as C
from oracle import torch_ref as T
from tests import wq_inputs as I
from tests.exact_arith import (BF16_1EM12, F32_1EM10, Fraction, e4m3_code, rn_bf16, rn_e4m3, rn_f32, round_to_format)

E4M3 = torch.float8_e4m3fn


def _codes(t):
    return t.view(torch.uint8)


def _bits32(t):
    return t.contiguous().view(torch.int32)


# ------------------------------------------------------------------ reference test-suite invariants
# tests/test_block_fp8_zero_block.py:38-75 of the reference, restated on both oracles.

@pytest.mark.parametrize("impl", ["torch", "c"])
def test_ref_zero_blocks_have_no_nan_and_positive_scale(impl):
    w = torch.zeros(256, 256, dtype=torch.bfloat16)
    w[0, 0] = 1.0
    q, s = T.block_fp8_ref(w, (128, 128)) if impl == "torch" else C.fp8_block_quant(w, (128, 128), 0)
    qf = q.float() if impl == "torch" else q.view(E4M3).float()
    assert not torch.isnan(qf).any() and not torch.isinf(qf).any()
    assert (s > 0).all()


@pytest.mark.parametrize("impl", ["torch", "c"])
def test_ref_zero_block_roundtrips_to_zero(impl):
    w = torch.zeros(128, 128, dtype=torch.bfloat16)
    q, s = T.block_fp8_ref(w, (128, 128)) if impl == "torch" else C.fp8_block_quant(w, (128, 128), 0)
    qf = q.float() if impl == "torch" else q.view(E4M3).float()
    assert ((qf * s.float()) == 0).all()


@pytest.mark.parametrize("impl", ["torch", "c"])
def test_ref_nonzero_blocks_roundtrip_error(impl):
    torch.manual_seed(0)
    w = torch.randn(256, 256, dtype=torch.float32).to(torch.bfloat16)
    q, s = T.block_fp8_ref(w, (128, 128)) if impl == "torch" else C.fp8_block_quant(w, (128, 128), 0)
    qf = q.float() if impl == "torch" else q.view(E4M3).float()
    assert not torch.isnan(qf).any()
    deq = qf * s.repeat_interleave(128, 0).repeat_interleave(128, 1).float()
    assert (deq - w.float()).abs().max() < 0.5


def test_ref_kat_dequant_bf16_scale():
    # tests/test_hf_to_megatron.py:345-358: linspace(-2,2) as e4m3, scale 2.0 -> exactly weight.bf16 * 2
    w = torch.linspace(-2, 2, 128 * 128).view(128, 128).to(E4M3)
    s = torch.tensor([[2.0]])
    want = w.to(torch.bfloat16) * 2
    assert I.same_bits(T.weight_dequant_bf16_scale_ref(w, s), want)
    assert I.same_bits(C.fp8_block_dequant(_codes(w), s, 128, 1), want)
    # a power-of-two scale makes both dequant variants agree
    assert I.same_bits(C.fp8_block_dequant(_codes(w), s, 128, 0), want)


# ------------------------------------------------------------------ hand-derived known answers

def test_zero_block_scale_bits_and_codes():
    w = torch.zeros(128, 256, dtype=torch.bfloat16)
    w[:, 128:] = -0.0
    for q, s in (C.fp8_block_quant(w, (128, 128), 0), tuple(map(lambda t: t, T.block_fp8_ref(w, (128, 128))))):
        q = _codes(q)
        # f32(bf16(1e-12)) / 448: bf16(1e-12) = 0x2B8D
        assert _bits32(s).tolist() == [[0x27212492, 0x27212492]]
        assert (q[:, :128] == 0x00).all() and (q[:, 128:] == 0x80).all()


def test_amax_element_maps_to_448():
    w = torch.zeros(128, 128, dtype=torch.bfloat16)
    w[3, 5], w[7, 9], w[1, 1] = 0.5, -0.5, 0.25
    for mode in (0, 1):
        q, s = C.fp8_block_quant(w, (128, 128), mode)
        assert q[3, 5] == 0x7E and q[7, 9] == 0xFE
        assert q[1, 1] == 0x76          # 224 = 1.75 * 2^7
        assert Fraction(s.item()) == rn_f32(Fraction(1, 2) / 448)


def test_mode1_floor_is_fp32_1e_10():
    w = torch.zeros(128, 128, dtype=torch.bfloat16)
    q, s = C.fp8_block_quant(w, (128, 128), 1)
    assert _bits32(s).item() == _bits32(torch.tensor([1e-10], dtype=torch.float32) / 448).item()
    assert (q == 0).all()


def _all_values_under(amax_bits: int):
    """[k*128, 128] bf16: every finite bf16 value with |x| <= amax, each 128-row block holding amax itself."""
    vals = I.finite_bf16_values()
    amax = torch.tensor([amax_bits], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    x = vals[vals.abs() <= amax]
    x = torch.cat([x, torch.zeros((-x.numel()) % (128 * 128), dtype=torch.bfloat16)]).view(-1, 128)
    x[::128, 0] = amax
    return x


def test_modes_differ_where_they_should():
    # division (mode 0) and reciprocal-multiply (mode 1) disagree on a few percent of (x, amax) pairs -
    # at rounding ties - and on none of them by more than one code; a mistake that collapses one mode
    # onto the other would make them agree everywhere
    w = _all_values_under(0x46FB)
    q0, s0 = C.fp8_block_quant(w, (128, 128), 0)
    q1, s1 = C.fp8_block_quant(w, (128, 128), 1)
    assert torch.equal(s0, s1)
    d = q0 != q1
    assert 0 < int(d.sum()) < w.numel() // 10
    assert ((q0[d].int() - q1[d].int()).abs() == 1).all()


def test_device_arithmetic_scale_is_a_reciprocal_multiply_for_every_amax():
    # mode 2 over all finite bf16 amax values: scale == RN(max(amax, floor) * RN(1/448)) in exact arithmetic, and
    # it differs from the quotient of mode 0 for a large share of them (a mode 2 that divides would pass nothing)
    bits = torch.arange(1, 0x7F80, 37, dtype=torch.int32)
    w = torch.zeros(bits.numel(), 4, dtype=torch.bfloat16)
    w[:, 1] = bits.to(torch.int16).view(torch.bfloat16)
    _, s2 = C.fp8_block_quant(w, (1, 4), 2)
    _, s0 = C.fp8_block_quant(w, (1, 4), 0)
    inv = rn_f32(Fraction(1, 448))
    n_diff = 0
    for a, got2, got0 in zip(w[:, 1].float().tolist(), s2[:, 0].tolist(), s0[:, 0].tolist()):
        a = max(Fraction(a), BF16_1EM12)
        assert Fraction(got2) == rn_f32(a * inv) and Fraction(got0) == rn_f32(a / 448)
        n_diff += got2 != got0
    assert n_diff > bits.numel() // 4


# ------------------------------------------------------------------ exact rational arithmetic, tiny blocks

def _exact_block_quant(w, bm, bn, mode):
    M, N = w.shape
    tm, tn = -(-M // bm), -(-N // bn)
    vals = [[Fraction(v) for v in row] for row in w.float().tolist()]
    neg0 = (w.view(torch.int16) == -32768).tolist()
    codes = [[0] * N for _ in range(M)]
    scales = [[None] * tn for _ in range(tm)]
    for bi in range(tm):
        for bj in range(tn):
            cells = [(i, j) for i in range(bi * bm, min(M, bi * bm + bm)) for j in range(bj * bn, min(N, bj * bn + bn))]
            amax = max(abs(vals[i][j]) for i, j in cells)
            if mode == 0:
                scale = rn_f32(max(amax, BF16_1EM12) / 448)
            elif mode == 2:     # torch's GPU evaluation of `/ 448`: multiply by RN(1/448)
                scale = rn_f32(max(amax, BF16_1EM12) * rn_f32(Fraction(1, 448)))
            else:
                scale = rn_f32(max(amax, F32_1EM10) / 448)
                inv = rn_f32(1 / scale)
            scales[bi][bj] = scale
            for i, j in cells:
                q = rn_f32(vals[i][j] / scale) if mode != 1 else rn_f32(vals[i][j] * inv)
                q = min(max(q, Fraction(-448)), Fraction(448))
                codes[i][j] = e4m3_code(rn_e4m3(q), negative_zero=(vals[i][j] < 0 or neg0[i][j]))
    return codes, scales


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_block_quant_matches_exact_arithmetic(mode):
    w = I.weights(10, 14, seed=11, std=0.05, outlier_p=0.05)
    w[0, 0] = -0.0
    w[4:8, 4:8] = 0          # an all-zero 4x4 block
    w[8:10, 0:4] *= 1e-30    # tiny values: floor active in mode 1, subnormal codes
    q, s = C.fp8_block_quant(w, (4, 4), mode)
    codes, scales = _exact_block_quant(w, 4, 4, mode)
    assert q.tolist() == codes
    assert [[Fraction(v) for v in row] for row in s.tolist()] == scales


# ------------------------------------------------------------------ C oracle == torch restatement

SHAPES = [(128, 128), (256, 384), (300, 200), (7, 7168), (1, 1), (129, 127), (4100, 3000)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("mode", [0, 1, 2])
def test_c_equals_torch_block_quant(shape, mode):
    w = I.zero_blocks(I.weights(*shape, seed=sum(shape)), 0.2, seed=1)
    q, s = C.fp8_block_quant(w, (128, 128), mode)
    if mode == 1:
        qr, sr = T.blockwise_cast_ref(w, (128, 128))
    else:
        qr, sr = T.block_fp8_ref(w, (128, 128), device_arith=(mode == 2))
    assert torch.equal(q, _codes(qr))
    assert torch.equal(_bits32(s), _bits32(sr))


@pytest.mark.parametrize("block", [(32, 32), (64, 128), (128, 64), (1, 128), (16, 48)])
def test_c_equals_torch_other_block_sizes(block):
    w = I.weights(200, 330, seed=2)
    for mode, ref in ((0, T.block_fp8_ref), (1, T.blockwise_cast_ref)):
        q, s = C.fp8_block_quant(w, block, mode)
        qr, sr = ref(w, block)
        assert torch.equal(q, _codes(qr)) and torch.equal(_bits32(s), _bits32(sr))


def test_c_equals_torch_strided_input():
    base = I.weights(512, 768, seed=4)
    for view in (base[:, 128:640], base.t(), base[::2, ::3], base[100:357, 5:700]):
        q, s = C.fp8_block_quant(view, (128, 128), 0)
        qr, sr = T.block_fp8_ref(view, (128, 128))
        assert torch.equal(q, _codes(qr)) and torch.equal(_bits32(s), _bits32(sr))


def test_c_equals_torch_special_blocks():
    blocks = [I.subnormal_block(seed=1), I.near_max_block(seed=2), I.near_max_block(seed=3, amax=3.0e38),
              I.near_max_block(seed=4, amax=1.2e-38), torch.zeros(128, 128, dtype=torch.bfloat16)]
    w = torch.cat(blocks, dim=1)
    for mode, ref in ((0, T.block_fp8_ref), (1, T.blockwise_cast_ref)):
        q, s = C.fp8_block_quant(w, (128, 128), mode)
        qr, sr = ref(w, (128, 128))
        assert torch.equal(q, _codes(qr)) and torch.equal(_bits32(s), _bits32(sr))


def test_c_equals_torch_every_bf16_value_against_many_amax():
    # the element function over its whole x domain for a spread of scales, incl. the bf16(1e-12) floor
    g = I.gen(9)
    amax_bits = torch.cat([torch.randint(1, 0x7F80, (24,), generator=g),
                           torch.tensor([1, 0x2B8C, 0x2B8D, 0x2B8E, 0x7F7F])])
    for ab in amax_bits.tolist():
        w = _all_values_under(ab)
        for mode, ref in ((0, T.block_fp8_ref), (1, T.blockwise_cast_ref)):
            q, s = C.fp8_block_quant(w, (128, 128), mode)
            qr, sr = ref(w, (128, 128))
            assert torch.equal(q, _codes(qr)) and torch.equal(_bits32(s), _bits32(sr)), (hex(ab), mode)


def test_nan_and_inf_blocks():
    w = I.weights(128, 384, seed=6)
    w[5, 5] = float("nan")
    w[9, 130] = float("inf")
    w[10, 131] = -float("inf")
    q, s = C.fp8_block_quant(w, (128, 128), 0)
    qr, sr = T.block_fp8_ref(w, (128, 128))
    qr = _codes(qr)
    # NaN block: scale NaN, every code a NaN code (sign unspecified)
    assert s[0, 0].isnan() and sr[0, 0].isnan()
    assert ((q[:, :128] & 0x7F) == 0x7F).all() and ((qr[:, :128] & 0x7F) == 0x7F).all()
    # Inf block: scale Inf; finite -> signed zero; Inf/Inf -> NaN code
    assert s[0, 1].isinf() and sr[0, 1].isinf()
    blk, blkr = q[:, 128:256].clone(), qr[:, 128:256].clone()
    for b in (blk, blkr):
        assert b[9, 2] & 0x7F == 0x7F and b[10, 3] & 0x7F == 0x7F
        b[9, 2] = b[10, 3] = 0
        assert ((b & 0x7F) == 0).all()
    assert torch.equal(blk, blkr)
    # untouched block is ordinary
    assert torch.equal(q[:, 256:], qr[:, 256:]) and torch.equal(_bits32(s[:, 2]), _bits32(sr[:, 2]))


@pytest.mark.parametrize("shape", [(64, 256), (3, 1000), (257, 129)])
def test_c_equals_torch_channel_and_tensor(shape):
    w = I.weights(*shape, seed=8)
    w[1] = 0
    for mode in (0, 2):
        q, s = C.fp8_channel_quant(w, mode)
        qr, sr = T.channel_fp8_ref(w, device_arith=(mode == 2))
        assert torch.equal(q, _codes(qr)) and torch.equal(_bits32(s), _bits32(sr)) and s.shape == sr.shape
        q, s = C.fp8_tensor_quant(w, mode)
        qr, sr = T.tensor_fp8_ref(w, device_arith=(mode == 2))
        assert torch.equal(q, _codes(qr)) and torch.equal(_bits32(s), _bits32(sr)) and s.shape == sr.shape


# ------------------------------------------------------------------ dequant

def test_dequant_all_codes_times_scales():
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8).repeat(128, 1)[:, :256]   # [128, 256]
    s = I.log_uniform_scales(1, 2, seed=3)
    for mode, ref in ((0, T.weight_dequant_ref), (1, T.weight_dequant_bf16_scale_ref)):
        got = C.fp8_block_dequant(codes, s, 128, mode)
        want = ref(codes.view(E4M3), s, 128)
        ok = ~want.isnan()
        assert torch.equal(got.isnan(), want.isnan())
        assert torch.equal(got[ok].view(torch.int16), want[ok].view(torch.int16))


@pytest.mark.parametrize("shape", [(256, 256), (300, 200), (7, 7168), (129, 1)])
def test_dequant_c_equals_torch(shape):
    x = I.fp8_codes(*shape, seed=shape[0])
    s = I.log_uniform_scales(-(-shape[0] // 128), -(-shape[1] // 128), seed=shape[1])
    for mode, ref in ((0, T.weight_dequant_ref), (1, T.weight_dequant_bf16_scale_ref)):
        assert I.same_bits(C.fp8_block_dequant(x, s, 128, mode), ref(x.view(E4M3), s, 128))


def test_dequant_exact_rational():
    x = I.fp8_codes(4, 40, seed=2)
    s = I.log_uniform_scales(1, 1, seed=5)
    got = C.fp8_block_dequant(x, s, 128, 0).float().tolist()
    got1 = C.fp8_block_dequant(x, s, 128, 1).float().tolist()
    xv = x.view(E4M3).float().tolist()
    sv = Fraction(s.item())
    for i in range(4):
        for j in range(40):
            assert Fraction(got[i][j]) == rn_bf16(rn_f32(Fraction(xv[i][j]) * sv))
            assert Fraction(got1[i][j]) == rn_bf16(rn_f32(Fraction(xv[i][j]) * rn_bf16(sv)))


def test_quant_dequant_roundtrip_error_bound():
    w = I.weights(512, 512, seed=12)
    q, s = C.fp8_block_quant(w, (128, 128), 0)
    d = C.fp8_block_dequant(q, s, 128, 0).float()
    step = s.repeat_interleave(128, 0).repeat_interleave(128, 1) * 32   # largest e4m3 spacing (at 448) is 32
    assert ((d - w.float()).abs() <= step / 2 * 1.01 + 1e-30).all()


def test_tensor_fp8_rounds_quotient_to_bf16_first():
    # tensor_fp8 divides by a 0-dim fp32 tensor, so torch keeps the quotient in bf16: two roundings.
    w = I.weights(6, 40, seed=21, std=0.05, outlier_p=0.02)
    q, s = C.fp8_tensor_quant(w)
    amax = max(abs(Fraction(v)) for row in w.float().tolist() for v in row)
    scale = rn_f32(max(amax, BF16_1EM12) / 448)
    assert Fraction(s.item()) == scale
    twice, once = 0, 0
    for i, row in enumerate(w.float().tolist()):
        for j, v in enumerate(row):
            q32 = rn_f32(Fraction(v) / scale)
            want = e4m3_code(rn_e4m3(min(max(rn_bf16(q32), Fraction(-448)), Fraction(448))), negative_zero=v < 0)
            assert q[i, j].item() == want
            twice += want != e4m3_code(rn_e4m3(min(max(q32, Fraction(-448)), Fraction(448))), negative_zero=v < 0)
    # the double rounding is observable on this sample (otherwise the test would not pin it)
    assert twice > 0


# ------------------------------------------------------------------ fp16 / fp32 weights

def _as_dtype(w, dt, seed):
    g = torch.Generator().manual_seed(seed)
    return (w.float() * (1 + 1e-3 * torch.randn(w.shape, generator=g))).to(dt)


@pytest.mark.parametrize("dt", [torch.float16, torch.float32])
@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("shape", [(256, 384), (300, 200), (7, 7168), (129, 127)])
def test_c_equals_torch_block_quant_other_dtypes(dt, mode, shape):
    x = _as_dtype(I.zero_blocks(I.weights(*shape, seed=sum(shape)), 0.2, seed=1), dt, 3)
    for view in (lambda t: t, lambda t: t.t()):
        q, s = C.fp8_block_quant(view(x), (128, 128), mode)
        qr, sr = T.blockwise_cast_ref(view(x), (128, 128)) if mode == 1 else T.block_fp8_ref(view(x), (128, 128), mode == 2)
        qr = _codes(qr)
        nan = (qr & 0x7F) == 0x7F
        assert torch.equal((q & 0x7F) == 0x7F, nan) and torch.equal(q[~nan], qr[~nan])
        assert torch.equal(_bits32(s), _bits32(sr))
        # an all-zero fp16 block divides 0 by 0 in the torch formulation (its 1e-12 floor rounds to 0 in fp16)
        if not (dt == torch.float16 and mode != 1):
            assert not nan.any()
        elif shape == (300, 200):
            assert nan.any()


def test_fp16_conversion_is_exact_for_every_value():
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.float16).view(-1, 64)
    finite = x.float().abs() < float("inf")
    x = torch.where(finite, x, torch.zeros_like(x))
    # mode 1 with a huge block: scale = amax / 448 with amax = 65504, codes = e4m3(x * (1 / scale))
    q, s = C.fp8_block_quant(x, (1024, 64), 1)
    qr, sr = T.blockwise_cast_ref(x, (1024, 64))
    assert torch.equal(q, _codes(qr)) and torch.equal(_bits32(s), _bits32(sr))


def test_fp32_floor_is_fp32_1e_12():
    w = torch.zeros(4, 4, dtype=torch.float32)
    w[0, 0] = 3e-13
    _, s0 = C.fp8_block_quant(w, (4, 4), 0)
    assert Fraction(s0.item()) == rn_f32(rn_f32(Fraction(1, 10 ** 12)) / 448)
    _, s2 = C.fp8_block_quant(w, (4, 4), 2)
    assert Fraction(s2.item()) == rn_f32(rn_f32(Fraction(1, 10 ** 12)) * rn_f32(Fraction(1, 448)))


# ------------------------------------------------------------------ power-of-two (UE8M0) scales: PARITY UNPINNED
# The arithmetic lives in sglang / DeepGEMM, which the reference does not vendor.  These tests pin what the
# mathematics fixes, and that the two restatements (literal log2 / ceil / pow chain, exponent arithmetic) agree.

def test_ue8m0_scale_is_the_smallest_power_of_two_not_below_amax_over_448_for_every_bf16_amax():
    bits = torch.arange(0, 0x7F80, dtype=torch.int32)
    n = bits.numel()
    w = torch.zeros(128, 128 * n, dtype=torch.bfloat16)
    w[0, ::128] = bits.to(torch.int16).view(torch.bfloat16)
    q, s = T.quant_weight_ue8m0_ref(w)
    qo, so = C.fp8_block_quant(w, (128, 128), 3)
    assert torch.equal(s.view(torch.int32), so.view(torch.int32)) and torch.equal(q.view(torch.uint8), qo)
    s64 = so.double().view(-1)
    amax = w[0, ::128].double().clamp(min=float(torch.tensor(1e-4, dtype=torch.float32)))
    mant, _ = torch.frexp(s64)
    assert (mant == 0.5).all()                                         # a power of two
    assert (s64 * 448 >= amax).all() and (s64 * 448 < 2 * amax).all()  # the smallest one that keeps |q| <= 448
    exact = amax == 448 * s64                                          # amax = 1.75 * 2^k: amax / 448 is itself a power of two
    assert int(exact.sum()) > 100


def test_ue8m0_literal_log2_ceil_pow_expression_for_every_bf16_amax():
    """sglang evaluates the scale as ``2 ** ceil(log2(amax / 448))`` in fp32; the C oracle (and the kernel) round the
    exponent up by bit manipulation.  The literal torch expression, evaluated here on all 32 639 finite non-zero bf16
    amax values, gives the oracle's scale bits for every one of them - fp32 log2 never lands on the wrong side of an
    integer for these inputs."""
    bits = torch.arange(1, 0x7F80, dtype=torch.int32)
    amax = bits.to(torch.int16).view(torch.bfloat16).float().clamp(1e-4)
    literal = torch.pow(2.0, torch.ceil(torch.log2(amax / 448.0)))
    w = torch.zeros(128, 128 * bits.numel(), dtype=torch.bfloat16)
    w[5, 3::128] = -bits.to(torch.int16).view(torch.bfloat16)
    _, so = C.fp8_block_quant(w, (128, 128), 3)
    assert torch.equal(literal.view(torch.int32), so.view(-1).view(torch.int32))


def test_ue8m0_codes_are_one_rounding_of_an_exact_scaling():
    w = I.zero_blocks(I.weights(300, 520, seed=3), 0.2, seed=1)
    w[200:, 300:] = I.subnormal_block(100, 220, seed=2)
    qo, so = C.fp8_block_quant(w, (128, 128), 3)
    q, s = T.quant_weight_ue8m0_ref(w)
    assert torch.equal(q.view(torch.uint8), qo) and torch.equal(s.view(torch.int32), so.view(torch.int32))
    full = T._expand_scale(so, 300, 520, 128).double()
    exact = w.double() / full                                           # a power-of-two divisor: exact in fp64 and fp32
    assert (exact.abs() <= 448).all()
    assert torch.equal(qo, C.f32_to_e4m3fn(exact.float()))              # codes = RNE of the exactly scaled value
    assert ((qo & 0x7F) <= 0x7E).all()
    deq = C.e4m3fn_to_f32(qo).double() * full
    step = full * torch.clamp(2.0 ** (torch.floor(torch.log2(exact.abs().clamp(min=2.0 ** -6))) - 3), min=2.0 ** -9)
    assert ((deq - w.double()).abs() <= step / 2).all()                 # within half an e4m3 step of the block
    zero = so[0, 4] if float(w[:128, 512:].abs().max()) == 0 else None
    assert so.min() >= 2.0 ** -22                                       # the 1e-4 floor: 1e-4 / 448 rounds up to 2^-22


def test_ue8m0_differs_from_the_plain_block_scale():
    w = I.weights(256, 256, seed=5)
    _, s0 = C.fp8_block_quant(w, (128, 128), 1)
    _, s3 = C.fp8_block_quant(w, (128, 128), 3)
    assert (s3 >= s0).all() and not torch.equal(s0, s3)


@pytest.mark.parametrize("dt", [torch.float16, torch.float32])
@pytest.mark.parametrize("device_arith", [False, True])
def test_channel_and_tensor_forms_other_dtypes(dt, device_arith):
    """fp16 / fp32 weights: the C oracle against the op-for-op torch restatement - the per-tensor quotient takes the
    weight's dtype (and, in the GPU evaluation, so does the divisor); rows are blocks of one row."""
    g = torch.Generator().manual_seed(3)
    for shape, std in (((37, 200), 0.05), ((128, 130), 1.0), ((5, 1000), 1e-3)):
        w = (torch.randn(shape, generator=g) * std).to(dt)
        for view in (lambda t: t, lambda t: t.t()):
            x = view(w)
            q, s = C.fp8_tensor_quant(x, 2 if device_arith else 0)
            qr, sr = T.tensor_fp8_ref(x, device_arith)
            assert torch.equal(q, qr.view(torch.uint8)) and torch.equal(s.view(torch.int32), sr.view(torch.int32))
            q, s = C.fp8_channel_quant(x, 2 if device_arith else 0)
            qr, sr = T.channel_fp8_ref(x, device_arith)
            assert torch.equal(q, qr.view(torch.uint8)) and torch.equal(s.view(torch.int32), sr.view(torch.int32))
    # fp32 weights round once: the per-tensor form equals one block spanning the tensor
    w = (torch.randn(64, 96, generator=g) * 0.3)
    q, s = C.fp8_tensor_quant(w, 0)
    qb, sb = C.fp8_block_quant(w, (64, 96), 0)
    assert torch.equal(q, qb) and torch.equal(s.view(torch.int32), sb.view(-1).view(torch.int32))
    # fp16 weights round twice.  Exact rational arithmetic on every element: scale = RN32(amax / 448),
    # code = e4m3(RN16(RN32(x / scale))); the sample must contain elements on which one rounding would differ
    f16 = lambda v: round_to_format(v, 11, -14)
    h = (torch.randn(1, 3000, generator=g) * 30).clamp(-100, 100).to(torch.float16)
    h[0, 0] = 100.25                                            # amax
    q, sc = C.fp8_tensor_quant(h, 0)
    scale = rn_f32(Fraction(100.25) / 448)
    assert Fraction(sc.item()) == scale
    differ = 0
    for v, code in zip(h[0].tolist(), q[0].tolist()):
        q32 = rn_f32(Fraction(v) / scale)
        assert code == e4m3_code(rn_e4m3(f16(q32)), negative_zero=(v < 0 and f16(q32) == 0)), v
        differ += rn_e4m3(f16(q32)) != rn_e4m3(q32)
    assert differ > 0
