"""Pins the INT4 part of the oracle.  The reference's first stage is a CUDA-only kernel with no test and
no CPU implementation, so it is pinned to its source text by exact rational arithmetic on small inputs,
closed-form special cases and invariants; the packing chain (torch primitives) is pinned op-for-op and by
its closed form."""

import pytest
import torch

from oracle import c_oracle as C
from oracle import torch_ref as T
from tests import wq_inputs as I
from tests.exact_arith import F32_1EM5, F32_ONE_SEVENTH, Fraction, rn_bf16, rn_f32, rne_int


def _exact_fake_quant_sym(w, gs):
    M, N = w.shape
    vals = [[Fraction(v) for v in row] for row in w.float().tolist()]
    q = [[0] * N for _ in range(M)]
    sc = [[None] * (N // gs) for _ in range(M)]
    for i in range(M):
        for g in range(N // gs):
            grp = vals[i][g * gs:(g + 1) * gs]
            amax = max(abs(v) for v in grp)
            scale = max(rn_f32(amax * F32_ONE_SEVENTH), F32_1EM5)     # multiply by RN(1/7), not divide by 7
            sc[i][g] = scale
            for k, v in enumerate(grp):
                q[i][g * gs + k] = rne_int(rn_f32(v / scale))
    return q, sc


@pytest.mark.parametrize("gs", [32, 128])
def test_fake_quant_sym_matches_exact_arithmetic(gs):
    w = I.weights(5, 2 * gs, seed=gs, std=0.02, outlier_p=0.02)
    w[1, :gs] = 0                       # floor 1e-5 active
    w[2, :gs] *= 1e-4                   # floor active with non-zero values
    q, s, z = C.int4_fake_quant(w, (1, gs), True)
    qe, se = _exact_fake_quant_sym(w, gs)
    assert [[int(v) for v in row] for row in q.float().tolist()] == qe
    assert [[Fraction(v) for v in row] for row in s.float().tolist()] == [[rn_bf16(v) for v in row] for row in se]
    assert (z == 0).all()
    qf, sf, _ = C.int4_fake_quant(w.float(), (1, gs), True)      # fp32 in / fp32 out keeps the fp32 scale
    assert [[Fraction(v) for v in row] for row in sf.tolist()] == se
    assert torch.equal(qf, q.float())


def test_fake_quant_multiply_by_one_seventh_not_divide_by_seven():
    # amax = 7 * 2^k: a division by 7 gives exactly 2^k, RN(amax * RN(1/7)) differs for some k - find the
    # convention from exact arithmetic and check the oracle follows the multiplication
    seen_diff = False
    for a in [0.0546875, 0.109375, 0.875, 1.75, 14.0, 0.0068359375, 0.013671875, 112.0, 0.4375, 3.5, 7.0, 28.0]:
        w = torch.zeros(1, 32, dtype=torch.bfloat16)
        w[0, 0] = a
        _, s, _ = C.int4_fake_quant(w.float(), (1, 32), True)
        mul = rn_f32(Fraction(a) * F32_ONE_SEVENTH)
        div = rn_f32(Fraction(a) / 7)
        assert Fraction(s.item()) == max(mul, F32_1EM5)
        seen_diff |= mul != div
    # generic values expose the difference
    w = I.weights(64, 32, seed=77, outlier_p=0).float()
    _, s, _ = C.int4_fake_quant(w, (1, 32), True)
    for i in range(64):
        amax = max(abs(Fraction(v)) for v in w[i].tolist())
        mul, div = rn_f32(amax * F32_ONE_SEVENTH), rn_f32(amax / 7)
        assert Fraction(s[i, 0].item()) == max(mul, F32_1EM5)
        seen_diff |= mul != div
    assert seen_diff


def test_fake_quant_invariants():
    w = I.weights(64, 1024, seed=5)
    q, s, _ = C.int4_fake_quant(w, (1, 128), True)
    qf = q.float()
    assert qf.abs().max() <= 7 and torch.equal(qf, qf.round())
    # the group's largest magnitude lands on +-7
    amax_pos = w.float().abs().view(64, 8, 128).argmax(dim=2)
    picked = qf.view(64, 8, 128).gather(2, amax_pos.unsqueeze(-1)).abs()
    assert (picked == 7).all()
    # reconstruction error at most half a step (of the fp32 scale; bf16-rounded scale adds 2^-9 relative)
    sf = s.float().repeat_interleave(128, dim=1)
    assert ((qf * sf - w.float()).abs() <= sf * (0.5 + 7 * 2 ** -8)).all()
    # zero group: scale is bf16(1e-5f), codes 0
    z = torch.zeros(2, 128, dtype=torch.bfloat16)
    q0, s0, _ = C.int4_fake_quant(z, (1, 128), True)
    assert (q0 == 0).all() and (s0.view(torch.int16) == 0x3728).all()


def _exact_fake_quant_asym(w, gs):
    M, N = w.shape
    vals = [[Fraction(v) for v in row] for row in w.float().tolist()]
    q = [[0] * N for _ in range(M)]
    sc, zp = [[None] * (N // gs) for _ in range(M)], [[None] * (N // gs) for _ in range(M)]
    f32_1_15 = rn_f32(Fraction(1, 15))
    for i in range(M):
        for g in range(N // gs):
            grp = vals[i][g * gs:(g + 1) * gs]
            vmax, vmin = max(grp), min(grp)
            scale = max(rn_f32(rn_f32(vmax - vmin) * f32_1_15), F32_1EM5)
            zero = min(max(-rne_int(rn_f32(vmin / scale)), 0), 15)
            sc[i][g], zp[i][g] = scale, zero
            for k, v in enumerate(grp):
                q[i][g * gs + k] = rne_int(rn_f32(v / scale)) + zero
    return q, sc, zp


def test_fake_quant_asym_matches_exact_arithmetic():
    w = I.weights(4, 64, seed=3, std=0.05).float()
    w[1] += 0.2           # all positive group: zero point clamps at 0
    w[2] -= 0.3           # all negative: clamps at 15
    q, s, z = C.int4_fake_quant(w, (1, 32), False)
    qe, se, ze = _exact_fake_quant_asym(w, 32)
    assert [[int(v) for v in row] for row in q.tolist()] == qe
    assert [[Fraction(v) for v in row] for row in s.tolist()] == se
    assert [[int(v) for v in row] for row in z.tolist()] == ze


@pytest.mark.parametrize("block", [(1, 32), (1, 128), (1, 64), (32, 1), (4, 8), (2, 16), (1, 256)])
@pytest.mark.parametrize("sym", [True, False])
def test_fake_quant_c_equals_torch(block, sym):
    w = I.weights(70, 300, seed=block[0] * 100 + block[1])      # ragged in both directions
    for x in (w, w.float(), w.t()):
        q, s, z = C.int4_fake_quant(x, block, sym)
        qr, sr, zr = T.fake_int4_quant_ref(x, block, sym)
        assert I.same_bits(q, qr) and I.same_bits(s, sr) and I.same_bits(z, zr)


def test_fake_quant_rejects_shapes_the_reference_kernels_mishandle():
    w = torch.zeros(64, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        C.int4_fake_quant(w, (1, 48), True)       # 48 % 32 != 0: TORCH_CHECK in the reference
    with pytest.raises(RuntimeError):
        C.int4_fake_quant(w, (2, 64), True)       # reference kernel would skip the second row


# ------------------------------------------------------------------ packing chain

def test_pack_to_int32_closed_form():
    g = I.gen(0)
    q = torch.randint(-8, 8, (9, 40), generator=g, dtype=torch.int32).to(torch.int8)
    words = T.pack_to_int32_ref(q, 4, sym=True)
    want = torch.zeros(9, 5, dtype=torch.int64)
    for j in range(8):
        want += (q[:, j::8].to(torch.int64) + 8) << (4 * j)
    want = torch.where(want >= 2 ** 31, want - 2 ** 32, want).to(torch.int32)     # int32 wrap-around
    assert torch.equal(words, want)
    # padding: 37 columns pad to 40 with zeros AFTER the +8 offset
    words = T.pack_to_int32_ref(q[:, :37], 4, sym=True)
    assert words.shape == (9, 5)
    assert (((words[:, 4].to(torch.int64) & 0xFFFFFFFF) >> 20) == 0).all()
    with pytest.raises(ValueError):
        T.pack_to_int32_ref(q, 9)
    with pytest.raises(ValueError):
        T.pack_to_int32_ref(q, 0)


def test_dequant_requant_is_identity_on_codes():
    # every code q in [-7, 7] and every bf16 scale the 1e-5 floor allows (0x3728 .. below Inf/7):
    # int8(round(clamp(bf16(bf16(q*s)/s)))) == q.  This is what lets the fused kernel skip the chain.
    sb = torch.arange(0x3728, 0x7C00, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    q = torch.arange(-7, 8, dtype=torch.float32).to(torch.bfloat16)
    d = q[None, :] * sb[:, None]
    r = torch.round(torch.clamp(d / sb[:, None], -128, 127)).to(torch.int8)
    assert torch.equal(r, q.to(torch.int8)[None, :].expand_as(r))
    assert int((d / sb[:, None] != q[None, :]).sum()) > 0      # the intermediate is NOT always q: rounding matters


@pytest.mark.parametrize("shape,gs", [((16, 256), 128), ((33, 768), 128), ((8, 2048), 128), ((24, 96), 32), ((8, 512), 64)])
@pytest.mark.parametrize("sym", [True, False])
def test_pack_layer_c_equals_torch(shape, gs, sym):
    if not sym and shape[0] % 8:
        pytest.skip("asymmetric zero-point packing needs M % 8 == 0 (reshape in the reference)")
    w = I.weights(*shape, seed=shape[1])
    w[0, :gs] = 0
    p, s, z = C.int4_pack_layer(w, gs, sym)
    pr, sr, zr = T.pack_layer_ref(w, gs, sym)
    assert torch.equal(p, pr) and I.same_bits(s, sr)
    assert (z is None and zr is None) if sym else torch.equal(z, zr)


def test_pack_layer_sym_equals_direct_formula():
    w = I.weights(32, 1024, seed=4)
    p, s, _ = C.int4_pack_layer(w, 128, True)
    q, s2, _ = C.int4_fake_quant(w, (1, 128), True)
    want = torch.zeros(32, 128, dtype=torch.int64)
    for j in range(8):
        want += (q[:, j::8].to(torch.int64) + 8) << (4 * j)
    want = torch.where(want >= 2 ** 31, want - 2 ** 32, want).to(torch.int32)
    assert torch.equal(p, want) and I.same_bits(s, s2)


def test_asym_dequant_requant_is_identity_on_small_codes():
    # the asymmetric chain of pack_layer: bf16(q - z) * s -> / s -> + z -> clamp to uint8 -> round, all in bf16, over
    # every code in [0, 17], every zero point and every positive bf16 scale below 2^121
    bits = torch.arange(0x0001, 0x7C00, dtype=torch.int32)
    sb = bits.to(torch.int16).view(torch.bfloat16)
    for q in range(18):
        for z in range(16):
            qv, zv = torch.full_like(sb, float(q)), torch.full_like(sb, float(z))
            r = ((qv - zv) * sb) / sb + zv
            assert (torch.round(torch.clamp(r, 0, 255)).to(torch.uint8) == q).all(), (q, z)
    # and it is not the identity everywhere above: the kernels must run the chain there
    big = torch.tensor([0x7F00], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    r = ((torch.full_like(big, 15.0) - 0) * big) / big
    assert not (torch.round(torch.clamp(r, 0, 255)) == 15).all()


def test_pack_layer_extreme_scales_where_the_chain_is_not_the_identity():
    # bf16(7 * scale) overflows to infinity for scales near 2^125: the chain then yields code 127 and the
    # packing sum carries into neighbouring nibbles.  Both oracles must agree on that corner too.
    w = I.near_max_block(8, 256, seed=3, amax=3.0e38)
    w[1] = I.near_max_block(1, 256, seed=4, amax=3.3895e38)[0]
    p, s, _ = C.int4_pack_layer(w, 128, True)
    pr, sr, _ = T.pack_layer_ref(w, 128, True)
    assert torch.equal(p, pr) and I.same_bits(s, sr)
    q, _, _ = C.int4_fake_quant(w, (1, 128), True)
    direct = torch.zeros(8, 32, dtype=torch.int64)
    for j in range(8):
        direct += (q[:, j::8].to(torch.int64) + 8) << (4 * j)
    direct = torch.where(direct >= 2 ** 31, direct - 2 ** 32, direct).to(torch.int32)
    assert not torch.equal(p, direct)      # the corner is real: the literal chain differs from the direct formula


# ------------------------------------------------------------------ INT4 -> bf16 and the QAT forward
# _dequantize_tensor's unpacking step is a third-party routine that is not available (parity unpinned against
# it); what is pinned: the bit layout is the inverse of pack_to_int32 (itself pinned above), and the arithmetic
# follows from exact rational arithmetic.

def test_int4_dequant_inverts_pack_to_int32_and_matches_exact_arithmetic():
    g = I.gen(31)
    codes = torch.randint(-8, 8, (6, 64), generator=g, dtype=torch.int32).to(torch.int8)
    packed = T.pack_to_int32_ref(codes, 4, sym=True)
    scale = I.weights(6, 2, seed=32, std=0.01).abs() + 1e-4
    got = C.int4_dequant(packed, scale, (6, 64), 32)
    assert I.same_bits(got, T.int4_dequant_ref(packed, scale, (6, 64), 32))
    want = [[rn_bf16(Fraction(int(codes[i, j])) * Fraction(scale[i, j // 32].float().item())) for j in range(64)]
            for i in range(6)]
    assert [[Fraction(v) for v in row] for row in got.float().tolist()] == want
    # nibble order: only element 8c+j set -> word c == (q+8) << 4j, all other nibbles hold the offset 8
    for j in range(8):
        one = torch.zeros(1, 32, dtype=torch.int8)
        one[0, 8 + j] = 5
        p = T.pack_to_int32_ref(one, 4, sym=True)
        d = C.int4_dequant(p, torch.ones(1, 1, dtype=torch.bfloat16), (1, 32), 32)
        assert d[0, 8 + j].item() == 5 and d.float().sum().item() == 5


@pytest.mark.parametrize("shape,gs", [((16, 256), 128), ((33, 768), 128), ((24, 96), 32), ((8, 512), 64)])
def test_int4_dequant_of_pack_layer_is_within_half_a_step(shape, gs):
    w = I.weights(*shape, seed=shape[0], outlier_p=0.01)
    packed, scale, _ = C.int4_pack_layer(w, gs, True)
    d = C.int4_dequant(packed, scale, shape, gs)
    assert I.same_bits(d, T.int4_dequant_ref(packed, scale, shape, gs))
    step = scale.float().repeat_interleave(gs, 1)
    assert ((d.float() - w.float()).abs() <= step * (0.5 + 7 * 2.0 ** -8) + d.float().abs() * 2.0 ** -8).all()


def _exact_ste(w, gs, device_arith):
    out = []
    for row in w.float().tolist():
        o = []
        for g in range(len(row) // gs):
            grp = [Fraction(v) for v in row[g * gs:(g + 1) * gs]]
            amax = max(abs(v) for v in grp)
            s = rn_f32(amax * F32_ONE_SEVENTH) if device_arith else rn_f32(amax / 7)
            s = max(s, F32_1EM5)
            for v in grp:
                q = min(max(rne_int(rn_f32(v / s)), -7), 7)
                o.append(rn_bf16(rn_f32(q * s)))
        out.append(o)
    return out


@pytest.mark.parametrize("device_arith", [False, True])
def test_fake_ste_matches_exact_arithmetic(device_arith):
    w = I.weights(6, 64, seed=41, std=0.02, outlier_p=0.03)
    w[1, :32] = 0
    w[2, :32] *= 1e-4
    got = C.int4_fake_ste(w, 32, int(device_arith))
    assert [[Fraction(v) for v in row] for row in got.float().tolist()] == _exact_ste(w, 32, device_arith)


@pytest.mark.parametrize("shape,gs", [((16, 256), 128), ((33, 768), 128), ((24, 96), 32), ((8, 512), 64), ((3, 100), 50)])
def test_fake_ste_c_equals_torch(shape, gs):
    w = I.weights(*shape, seed=shape[1], outlier_p=0.01)
    w[0, :gs] = 0
    differ = False
    for dev in (False, True):
        got = C.int4_fake_ste(w, gs, int(dev))
        assert I.same_bits(got, T.fake_int4_ste_ref(w, gs, device_arith=dev))
    big = I.weights(256, 1024, seed=5)
    assert not I.same_bits(C.int4_fake_ste(big, 128, 0), C.int4_fake_ste(big, 128, 1))


def test_fake_ste_is_idempotent_up_to_scale_rounding_and_bounded():
    w = I.weights(64, 1024, seed=6)
    y = C.int4_fake_ste(w, 128, 1)
    amax = w.float().view(64, 8, 128).abs().amax(-1, keepdim=True)
    step = (amax / 7).clamp(min=1e-5)
    assert ((y.float().view(64, 8, 128) - w.float().view(64, 8, 128)).abs() <= step * 0.5 * 1.02 + amax * 2.0 ** -8).all()
    # at most 15 distinct values per group
    assert max(len(set(r)) for r in y.float().view(-1, 128).tolist()) <= 15


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("gs", [128, 32, 24, 1, -1])
def test_int4_dequant_any_c_equals_torch(dt, gs):
    # the inputs the reference's _dequantize_tensor accepts beyond bf16 scales and whole groups of 8: other scale
    # dtypes (converted with .to(float32)), one scale per element (group_size <= 0), rows not a multiple of 8 long
    g = I.gen(gs + 200)
    M, N = 9, 96 if gs in (24, 32) else 128
    if gs in (1, -1):
        N = 52                                                      # ragged: 7 words per row, the last one cut
    packed = torch.randint(-2 ** 31, 2 ** 31 - 1, (M, -(-N // 8)), generator=g, dtype=torch.int64).to(torch.int32)
    group = gs if gs > 0 else 1
    scale = (torch.rand(M, N // group, generator=g) * 0.02 + 1e-4).to(dt)
    want = T.int4_dequant_ref(packed, scale, (M, N), gs)
    got = C.int4_dequant_any(packed, scale, (M, N), gs)
    assert I.same_bits(got, want)
    if dt == torch.bfloat16 and gs in (128, 32):
        assert I.same_bits(got, C.int4_dequant(packed, scale, (M, N), gs))


def test_int4_dequant_fp32_scale_rounds_twice():
    # fp32 scale: (int8 * scale) is rounded to fp32 and then to bf16.  With scale = RN(m / 3) for a bf16 midpoint m the
    # exact product 3 * scale lies a hair off m, the fp32 rounding lands ON m and the tie then goes to even - a single
    # rounding of the exact product would go to the nearer neighbour instead.
    from fractions import Fraction

    from tests import exact_arith as X

    word = 0xBBBBBBBB - (1 << 32)                                  # eight nibbles 0xB: q = 3
    packed = torch.tensor([[word]], dtype=torch.int32)
    hits = 0
    for k in range(64):
        mid = (1 + (2 * k + 1) * 2.0 ** -8) * 2.0 ** (k % 5 - 2)
        s = torch.tensor([[mid / 3]], dtype=torch.float32)
        got = C.int4_dequant_any(packed, s, (1, 8), 8)
        exact = 3 * Fraction(float(s))
        twice = X.rn_bf16(X.rn_f32(exact))
        if exact == Fraction(mid):                                  # m divisible by 3: nothing to round
            continue
        assert X.rn_f32(exact) == Fraction(mid)
        assert all(Fraction(float(v)) == twice for v in got[0])
        assert I.same_bits(got, T.int4_dequant_ref(packed, s, (1, 8), 8))
        hits += twice != X.rn_bf16(exact)
    assert hits >= 16


@pytest.mark.parametrize("sym", [True, False])
def test_fake_quant_fp64_converts_to_fp32_on_load(sym):
    # the reference dispatches float, double and bfloat16 (fake_int4_quant_cuda.cu:352) and casts each element to
    # float first (:70): an fp64 input gives the fp32 input's codes, stored as doubles
    g = I.gen(5)
    x64 = torch.randn(8, 256, generator=g, dtype=torch.float64) * 0.02
    q, s, z = C.int4_fake_quant(x64, (1, 128), sym)
    q32, s32, z32 = C.int4_fake_quant(x64.float(), (1, 128), sym)
    assert q.dtype == torch.float64 and torch.equal(q, q32.double()) and torch.equal(s, s32.double())
    if not sym:
        assert torch.equal(z, z32.double())
