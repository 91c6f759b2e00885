"""Seeded random shapes, views, block sizes and modes through every kernel family against the CPU oracle."""

import random

import pytest
import torch

import slime_amd
from oracle import c_oracle as C
from tests import wq_inputs as I

pytestmark = pytest.mark.gpu
E4M3 = torch.float8_e4m3fn
ARITH = {0: "cpu", 2: "device"}


def _view(rng, t):
    """A random view of t (possibly t itself): column / row slices, row strides, transposes."""
    kind = rng.choice(["same", "cols", "rows", "stride", "t", "cols8"])
    M, N = t.shape
    if kind == "cols" and N > 3:
        a = rng.randrange(0, N // 2)
        return t[:, a:rng.randrange(a + 1, N + 1)]
    if kind == "cols8" and N > 24:
        a = 8 * rng.randrange(0, N // 16)
        return t[:, a:a + 8 * rng.randrange(1, (N - a) // 8 + 1)]
    if kind == "rows" and M > 3:
        a = rng.randrange(0, M // 2)
        return t[a:rng.randrange(a + 1, M + 1)]
    if kind == "stride" and M > 2:
        return t[::2]
    if kind == "t":
        return t.t()
    return t


@pytest.mark.parametrize("seed", range(6))
def test_fp8_block_quant_random(cuda, seed):
    rng = random.Random(1000 + seed)
    for _ in range(12):
        M, N = rng.randrange(1, 700), rng.randrange(1, 900)
        w = I.zero_blocks(I.weights(M, N, seed=rng.randrange(1 << 30), outlier_p=0.01), 0.15, seed=seed)
        block = rng.choice([(128, 128)] * 3 + [(64, 64), (32, 128), (128, 32), (1, 128), (16, 48), (256, 64)])
        mode = rng.choice([0, 1, 2])
        wg = w.to(cuda)
        r1, r2 = random.Random(seed * 77 + M), random.Random(seed * 77 + M)
        wv, gv = _view(r1, w), _view(r2, wg)
        if mode == 1:
            q, s = slime_amd.blockwise_cast_to_fp8_triton(gv, block)
        else:
            with slime_amd.torch_arithmetic(ARITH[mode]):
                q, s = slime_amd.block_fp8(gv, block)
        qo, so = C.fp8_block_quant(wv, block, mode)
        assert torch.equal(q.cpu().view(torch.uint8), qo), (M, N, block, mode, tuple(wv.shape), wv.stride())
        assert torch.equal(s.cpu().view(torch.int32), so.view(torch.int32)), (M, N, block, mode)


@pytest.mark.parametrize("seed", range(4))
def test_fp8_dequant_random(cuda, seed):
    rng = random.Random(2000 + seed)
    for _ in range(12):
        M, N = rng.randrange(1, 700), rng.randrange(1, 1500)
        block = rng.choice([128, 128, 64, 32, 256, 48])
        x = I.fp8_codes(M, N, seed=rng.randrange(1 << 30))
        s = I.log_uniform_scales(-(-M // block), -(-N // block), seed=rng.randrange(1 << 30))
        for mode in (0, 1):
            y = slime_amd.fp8._dequant(x.to(cuda).view(E4M3), s.to(cuda), block, mode, torch.bfloat16, "random")
            assert I.same_bits(y.cpu(), C.fp8_block_dequant(x, s, block, mode)), (M, N, block, mode)


@pytest.mark.parametrize("seed", range(4))
def test_int4_random(cuda, seed):
    rng = random.Random(3000 + seed)
    for _ in range(10):
        gs = rng.choice([32, 64, 128, 128, 128, 96, 256])
        M, G = rng.randrange(1, 400), rng.randrange(1, 24)
        N = gs * G
        w = I.weights(M, N, seed=rng.randrange(1 << 30), outlier_p=0.01)
        if rng.random() < 0.3:
            w = w + 0.05                                  # one-sided groups for the asymmetric form
        w[rng.randrange(M), :gs] = 0
        sym = rng.random() < 0.5
        r1, r2 = random.Random(seed * 91 + M), random.Random(seed * 91 + M)
        wv, gv = _view(r1, w), _view(r2, w.to(cuda))
        bn = gs if wv.shape[1] % gs == 0 else 32
        q, s, z = slime_amd.fake_int4_quant_cuda(gv, (1, bn), sym)
        qo, so, zo = C.int4_fake_quant(wv, (1, bn), sym)
        assert I.same_bits(q.cpu(), qo) and I.same_bits(s.cpu(), so) and I.same_bits(z.cpu(), zo), (M, N, gs, sym, wv.stride())
        if gs % 32 == 0 and (sym or M % 8 == 0):
            p, sc, pz = slime_amd.pack_layer(w.to(cuda), gs, sym)
            po, so2, pzo = C.int4_pack_layer(w, gs, sym)
            assert torch.equal(p.cpu(), po) and I.same_bits(sc.cpu(), so2), (M, N, gs, sym)
            assert (pz is None and pzo is None) or torch.equal(pz.cpu(), pzo)
            if sym:
                d = slime_amd.dequantize_int4(p, sc, (M, N), gs)
                assert I.same_bits(d.cpu(), C.int4_dequant(po, so2, (M, N), gs))
        if gs in (32, 64, 128):
            for div7, arith in ((0, "cpu"), (1, "device")):
                with slime_amd.torch_arithmetic(arith):
                    y = slime_amd.fake_int4_quantization_ste(w.to(cuda), gs)
                assert I.same_bits(y.cpu(), C.int4_fake_ste(w, gs, div7)), (M, N, gs, arith)
