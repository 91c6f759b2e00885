"""Random shapes, strides, storage offsets, block sizes, dtypes and value ranges through the per-tensor functions, each
case against the CPU oracle (bit-exact; NaN-ness where the reference leaves a NaN's bits open).  The fixed-shape tests name
the cases the reference's configurations fix; this file sweeps what lies between them."""

import zlib

import pytest
import torch

import slime_amd
from oracle import c_oracle as C
from slime_amd import arith
from tests import wq_inputs as I

pytestmark = pytest.mark.gpu
E4M3 = torch.float8_e4m3fn


def same_or_nan(a, b):
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    na, nb = a.isnan(), b.isnan()
    return bool(torch.equal(na, nb)) and I.same_bits(torch.where(na, torch.zeros_like(a), a), torch.where(nb, torch.zeros_like(b), b))


def same_codes(q, qo):
    nan_o = (qo & 0x7F) == 0x7F
    return bool(torch.equal((q & 0x7F) == 0x7F, nan_o)) and bool(torch.equal(q[~nan_o], qo[~nan_o]))


def codes(t):
    return t.cpu().contiguous().view(torch.uint8)


def bits32(t):
    return t.cpu().contiguous().view(torch.int32)


class Draw:
    """Seeded draws: r(a, b) an integer in [a, b], pick(xs) one of xs."""

    def __init__(self, seed):
        self.g = torch.Generator().manual_seed(seed)

    def r(self, a, b):
        return int(torch.randint(a, b + 1, (1,), generator=self.g))

    def pick(self, xs):
        return xs[self.r(0, len(xs) - 1)]

    def dim(self, big):
        """A dimension up to ``big``: tiny, a multiple of 128, a multiple of 8, just past a multiple of 128, or anything."""
        k = self.r(0, 5)
        if k == 0:
            return self.r(1, 17)
        if k == 1:
            return 128 * self.r(1, big // 128)
        if k == 2:
            return 8 * self.r(1, big // 8)
        if k == 3:
            return 128 * self.r(1, max(big // 128 - 1, 1)) + self.pick([1, 7, 8, 64, 127])
        return self.r(1, big)

    def values(self, M, N, dtype):
        """Normal values at one of five magnitudes (down to subnormal results), sometimes with outliers, all-zero blocks or
        one Inf / NaN."""
        tiny = 1e-30 if dtype != torch.float16 else 1e-6
        w = torch.randn(M, N, generator=self.g) * self.pick([0.02, 1.0, 1e-6, 300.0, tiny])
        if self.r(0, 3) == 0:
            w[torch.rand(M, N, generator=self.g) < 0.01] *= 50
        if self.r(0, 4) == 0:
            w = I.zero_blocks(w, 0.3, seed=self.r(0, 99))
        if self.r(0, 9) == 0 and M * N > 4:
            w.view(-1)[self.r(0, M * N - 1)] = self.pick([float("inf"), float("-inf"), float("nan")])
        return w.to(dtype)

    def strided(self, w_cpu, cuda):
        """-> (host view, device view) of the same values with the same strides and storage offset: contiguous, a window of
        a larger matrix, every second column, or a transposed layout."""
        M, N = w_cpu.shape
        how = self.r(0, 4)
        if how <= 1:
            return w_cpu, w_cpu.to(cuda)
        if how == 2:
            pad_rows, pad_cols, off = self.r(0, 9), self.r(0, 9), self.r(0, 5)
            base = torch.zeros(M + pad_rows, N + pad_cols + off, dtype=w_cpu.dtype)
            base[:M, off:off + N] = w_cpu
            return base[:M, off:off + N], base.to(cuda)[:M, off:off + N]
        if how == 3:
            base = torch.zeros(M, 2 * N + 1, dtype=w_cpu.dtype)
            base[:, 1::2] = w_cpu
            return base[:, 1::2], base.to(cuda)[:, 1::2]
        t = w_cpu.t().contiguous()
        return t.t(), t.to(cuda).t()


def case_fp8_block(seed, cuda):
    d = Draw(seed)
    M, N = d.dim(700), d.dim(3000)
    dtype = d.pick([torch.bfloat16] * 4 + [torch.float32, torch.float16])
    block = d.pick([(128, 128)] * 4 + [(64, 32), (32, 64), (128, 64), (16, 16), (100, 60), (1, 128), (128, 1), (256, 256)])
    mode = d.pick([0, 1, 2, 3])
    if mode == 3:                                   # the power-of-two requantiser takes bf16 and 128 x 128 only
        dtype, block = torch.bfloat16, (128, 128)
    wc, wg = d.strided(d.values(M, N, dtype), cuda)
    if mode == 1:
        q, s = slime_amd.blockwise_cast_to_fp8_triton(wg, block)
    elif mode == 3:
        q, s = slime_amd.quant_weight_ue8m0(wg, block)
    else:
        with slime_amd.torch_arithmetic({0: "cpu", 2: "device"}[mode]):
            q, s = slime_amd.block_fp8(wg, block)
    qo, so = C.fp8_block_quant(wc, block, mode)
    what = (M, N, dtype, block, mode, wc.stride())
    assert same_codes(codes(q), qo), what
    ok = ~so.isnan()
    assert torch.equal(bits32(s)[ok], bits32(so)[ok]) and bool(s.cpu().isnan()[~ok].all()), what


def case_fp8_row_tensor(seed, cuda):
    d = Draw(seed)
    M, N = d.dim(700), d.dim(3000)
    dtype = d.pick([torch.bfloat16] * 4 + [torch.float32, torch.float16])
    mode = d.pick([0, 2])
    wc, wg = d.strided(d.values(M, N, dtype), cuda)
    with slime_amd.torch_arithmetic({0: "cpu", 2: "device"}[mode]):
        if d.r(0, 1):
            (q, s), (qo, so) = slime_amd.channel_fp8(wg), C.fp8_channel_quant(wc, mode)
        else:
            (q, s), (qo, so) = slime_amd.tensor_fp8(wg), C.fp8_tensor_quant(wc, mode)
    what = (M, N, dtype, mode, wc.stride())
    assert same_codes(codes(q), qo), what
    ok = ~so.isnan().reshape(-1)
    assert torch.equal(bits32(s).reshape(-1)[ok], bits32(so).reshape(-1)[ok]), what


def case_fp8_dequant(seed, cuda):
    d = Draw(seed)
    M, N = d.dim(700), d.dim(3000)
    block = d.pick([128] * 4 + [64, 32, 100, 256, 8, 1])
    x = torch.randint(0, 256, (M, N), generator=d.g, dtype=torch.int32).to(torch.uint8)          # every code, the two NaNs included
    s = torch.exp(torch.empty(-(-M // block), -(-N // block)).uniform_(-20, 5, generator=d.g))
    if d.r(0, 5) == 0:
        s.view(-1)[0] = d.pick([0.0, float("inf"), 1e-40, 3e38])
    out = d.pick([torch.bfloat16, torch.bfloat16, torch.float32, torch.float16])
    xg, sg = x.to(cuda).view(E4M3), s.to(cuda)
    if d.r(0, 3) == 0 and out == torch.bfloat16:
        y, yo = slime_amd.weight_dequant_bf16_scale(xg, sg, block), C.fp8_block_dequant(x, s, block, 1)
    else:
        y = slime_amd.block_quant_dequant(xg, sg, [block, block], out)
        f = C.e4m3fn_to_f32(x) * s.repeat_interleave(block, 0)[:M].repeat_interleave(block, 1)[:, :N]
        yo = C.fp8_block_dequant(x, s, block, 0) if out == torch.bfloat16 else (f if out == torch.float32 else C.f32_to_f16(f))
    assert same_or_nan(y.cpu(), yo), (M, N, block, out)


def case_int4(seed, cuda):
    """pack_layer (symmetric and asymmetric), its inverse, and the QAT forward on the same weights."""
    d = Draw(seed)
    group = d.pick([128, 128, 64, 32])
    sym = bool(d.r(0, 1))
    M = 8 * d.r(1, 90) if not sym or d.r(0, 1) else d.dim(700)          # zero points pack eight rows to a word
    N = group * d.r(1, 2048 // group)
    w = torch.nan_to_num(d.values(M, N, torch.bfloat16), nan=0.0, posinf=1.0, neginf=-1.0)
    got = slime_amd.pack_layer(w.to(cuda), group, sym)
    po, so, zo = C.int4_pack_layer(w, group, sym)
    what = (M, N, group, sym)
    assert torch.equal(got[0].cpu(), po), what
    assert I.same_bits(got[1].cpu(), so), what
    if sym:
        y = slime_amd.dequantize_int4(got[0], got[1], (M, N), group)
        assert I.same_bits(y.cpu(), C.int4_dequant(po, so, (M, N), group)), what
    else:
        assert torch.equal(got[2].cpu(), zo), what
    y = slime_amd.fake_int4_quantization_ste(w.to(cuda), group)
    assert I.same_bits(y.cpu(), C.int4_fake_ste(w, group, arith.div7_rule())), what


def case_fake_int4(seed, cuda):
    d = Draw(seed)
    M, N = d.dim(500), d.dim(2000)
    block = d.pick([(1, 128), (1, 128), (1, 32), (1, 64), (1, 96), (32, 1), (16, 16), (4, 8), (2, 32)])
    dtype = d.pick([torch.bfloat16, torch.bfloat16, torch.float32])
    sym = bool(d.r(0, 1))
    w = torch.nan_to_num(d.values(M, N, dtype), nan=0.0, posinf=1.0, neginf=-1.0)
    wc, wg = d.strided(w, cuda)
    q, sc, zp = slime_amd.fake_int4_quant_cuda(wg, block, sym)
    qo, sco, zpo = C.int4_fake_quant(wc, block, sym)
    what = (M, N, block, dtype, sym, wc.stride())
    assert I.same_bits(q.cpu(), qo), what
    assert I.same_bits(sc.cpu(), sco) and I.same_bits(zp.cpu(), zpo), what


def case_delta(seed, cuda):
    """new ^ old, the count of changed bytes, adler32 of the new bytes and the snapshot update, in one pass."""
    d = Draw(seed)
    dtype = d.pick([torch.bfloat16, torch.uint8, torch.float32, torch.int32])
    n = d.pick([d.r(1, 64), d.r(1, 100000), 256 * d.r(1, 4000), 16 * d.r(1, 50000) + d.pick([0, 2, 4, 8])])
    nbytes = n * torch.empty((), dtype=dtype).element_size()
    new = torch.randint(0, 256, (nbytes,), generator=d.g, dtype=torch.int32).to(torch.uint8)
    old = new.clone()
    if d.r(0, 3):
        idx = torch.randint(0, nbytes, (max(1, nbytes // d.pick([2, 100, 10000])),), generator=d.g)
        old[idx] ^= 0x5A
    new_gpu, old_gpu = new.to(cuda).view(dtype), old.to(cuda)
    update = bool(d.r(0, 1))
    diff, result = slime_amd.delta.xor_diff(new_gpu, old_gpu, update_snapshot=update)
    assert torch.equal(diff.cpu().reshape(-1), new ^ old), (n, dtype)
    changed, adler = result.cpu().tolist()
    assert changed == int((new != old).sum()) and adler == zlib.adler32(new.numpy().tobytes()), (n, dtype)
    assert torch.equal(old_gpu.cpu(), new if update else old), (n, dtype, update)


# ---------------------------------------------------------------------------------- one launch over many tensors
# The many-tensor forms against the per-tensor functions above (which the first half of this file holds to the oracle):
# lists short enough for the searched descriptors and long enough for the per-item tables, ragged members, repeats.


def _weight_list(d, cuda, cols, rows, lo=1, hi=90):
    n = d.pick([d.r(lo, 6), d.r(lo, hi)])
    return [d.values(d.pick(rows), d.pick(cols), torch.bfloat16).nan_to_num(0.0, 1.0, -1.0).to(cuda) for _ in range(n)]


def case_fp8_plans(seed, cuda):
    d = Draw(seed)
    ws = _weight_list(d, cuda, [128, 256, 384, 200, 520, 7, 1000], [1, 7, 128, 129, 256, 300])
    if d.r(0, 2) == 0:
        ws[0] = d.strided(ws[0].cpu(), cuda)[1]
    block = d.pick([(128, 128), (128, 128), (64, 32), (100, 60)])
    mode = d.pick([0, 1, 2])
    outs = slime_amd.Fp8QuantPlan(ws, block, mode).run()
    for k, (w, (q, s)) in enumerate(zip(ws, outs)):
        if mode == 1:
            qo, so = slime_amd.blockwise_cast_to_fp8_triton(w, block)
        else:
            with slime_amd.torch_arithmetic({0: "cpu", 2: "device"}[mode]):
                qo, so = slime_amd.block_fp8(w, block)
        assert torch.equal(q.view(torch.uint8), qo.view(torch.uint8)) and I.same_bits(s, so), (k, tuple(w.shape), block, mode)
    if block[0] == block[1]:
        out_dtype = d.pick([torch.bfloat16, torch.float32])
        ys = slime_amd.Fp8DequantPlan([q for q, _ in outs], [s for _, s in outs], block[0], 0, out_dtype).run()
        for k, ((q, s), y) in enumerate(zip(outs, ys)):
            assert I.same_bits(y, slime_amd.block_quant_dequant(q, s, list(block), out_dtype)), (k, tuple(q.shape), block, out_dtype)


def case_int4_plans(seed, cuda):
    d = Draw(seed)
    group = d.pick([128, 128, 64, 32])
    sym = bool(d.r(0, 1))
    ws = _weight_list(d, cuda, [group * k for k in (1, 2, 3, 8, 11)], [8, 16, 128, 136, 304] + ([1, 7, 129] if sym else []))
    outs = slime_amd.Int4PackPlan(ws, group, sym).run()
    for k, (w, got) in enumerate(zip(ws, outs)):
        want = [v for v in slime_amd.pack_layer(w, group, sym) if v is not None]
        assert len(got) == len(want) and all(I.same_bits(a, b) for a, b in zip(got, want)), (k, tuple(w.shape), group, sym)
    if sym:
        ys = slime_amd.Int4DequantPlan([o[0] for o in outs], [o[1] for o in outs], [w.shape for w in ws], group).run()
        for k, (w, o, y) in enumerate(zip(ws, outs, ys)):
            assert I.same_bits(y, slime_amd.dequantize_int4(o[0], o[1], w.shape, group)), (k, tuple(w.shape), group)
    many = slime_amd.fake_int4_quantization_ste_many(ws, group)
    plan = slime_amd.Int4StePlan(ws, group).run()
    for k, (w, a, b) in enumerate(zip(ws, many, plan)):
        want = slime_amd.fake_int4_quantization_ste(w, group)
        assert I.same_bits(a, want) and I.same_bits(b, want), (k, tuple(w.shape), group)


def case_grouped_weights(seed, cuda):
    """The stacked form of a grouped linear's experts, twice: the second time every expert lives somewhere else."""
    d = Draw(seed)
    M, N = d.pick([128, 256, 384, 200, 7]), d.pick([128, 256, 520, 1000, 132])
    E = d.r(1, 12)
    block = d.pick([(128, 128), (128, 128), (64, 32)])
    ue8m0 = block == (128, 128) and bool(d.r(0, 1))
    for sync in range(2):
        ws = [d.values(M, N, torch.bfloat16).nan_to_num(0.0, 1.0, -1.0).to(cuda) for _ in range(E)]
        if d.r(0, 1):                                   # chunk views of one fused tensor
            ws = list(torch.cat(ws, dim=0).chunk(E, dim=0))
        q, s = slime_amd.quantize_grouped_weights(ws, block, ue8m0)
        for e, w in enumerate(ws):
            qo, so = slime_amd.quant_weight_ue8m0(w, block) if ue8m0 else slime_amd.blockwise_cast_to_fp8_triton(w, block)
            assert torch.equal(q[e].view(torch.uint8), qo.view(torch.uint8)) and I.same_bits(s[e], so), (sync, e, M, N, E, block, ue8m0)


def case_delta_many(seed, cuda):
    d = Draw(seed)
    n = d.pick([d.r(1, 5), d.r(1, 80)])
    news, olds = [], []
    for _ in range(n):
        nbytes = d.pick([d.r(1, 64), d.r(1, 70000), 256 * d.r(1, 300), 16384 * d.r(1, 8)])
        new = torch.randint(0, 256, (nbytes,), generator=d.g, dtype=torch.int32).to(torch.uint8)
        old = new.clone()
        if d.r(0, 2):
            old[torch.randint(0, nbytes, (max(1, nbytes // d.pick([2, 100, 10000])),), generator=d.g)] ^= 0xA5
        news.append(new.to(cuda))
        olds.append(old.to(cuda))
    want = [slime_amd.delta.xor_diff(a, b.clone()) for a, b in zip(news, olds)]
    diffs, results = slime_amd.delta.xor_diff_many(news, [o.clone() for o in olds])
    plan = slime_amd.delta.XorDiffPlan(news, [o.clone() for o in olds], xxh3=True)
    p_diffs, p_results = plan.run(update_snapshot=True)
    digests = plan.hexdigests()
    for k, (dw, rw) in enumerate(want):
        assert torch.equal(diffs[k], dw) and torch.equal(results[k], rw), (k, n)
        assert torch.equal(p_diffs[k], dw) and torch.equal(p_results[k], rw) and torch.equal(plan.olds[k], news[k]), (k, n)
        changed = int(rw[0])
        assert digests[k] == (slime_amd.delta.xxh3_128(news[k]) if changed else None), (k, n)


CASES = {"fp8_block": case_fp8_block, "fp8_row_tensor": case_fp8_row_tensor, "fp8_dequant": case_fp8_dequant, "int4": case_int4,
         "fake_int4": case_fake_int4, "delta": case_delta, "fp8_plans": case_fp8_plans, "int4_plans": case_int4_plans,
         "grouped_weights": case_grouped_weights, "delta_many": case_delta_many}


@pytest.mark.parametrize("seed", range(16))
@pytest.mark.parametrize("kind", list(CASES))
def test_random_case(cuda, kind, seed):
    CASES[kind](seed, cuda)
