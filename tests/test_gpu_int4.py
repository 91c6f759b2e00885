"""HIP INT4 kernels (through the C ABI) against the CPU oracle: bit-exact words, codes and scales."""

import os

import pytest
import torch

import slime_amd
from oracle import c_oracle as C
from tests import wq_inputs as I

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _check_pack(w, cuda, gs=128):
    p, s, z = slime_amd.pack_layer(w.to(cuda), gs, True)
    assert z is None and p.dtype == torch.int32 and s.dtype == torch.bfloat16
    assert p.is_contiguous() and s.is_contiguous()
    po, so, _ = C.int4_pack_layer(w, gs, True)
    assert p.shape == po.shape and s.shape == so.shape
    nbad = int((p.cpu() != po).sum())
    assert nbad == 0, f"{nbad} packed-word mismatches"
    assert I.same_bits(s.cpu(), so)


@pytest.mark.parametrize("shape", [(768, 2048), (2048, 768), (16, 256), (33, 768), (1, 128), (7, 7168), (1000, 2560)])
def test_pack_layer_g128(cuda, shape):
    w = I.weights(*shape, seed=shape[1])
    w[0, :128] = 0
    _check_pack(w, cuda)


@pytest.mark.parametrize("gs,shape", [(32, (24, 96)), (32, (768, 2048)), (64, (8, 512)), (64, (333, 1024)),
                                      (256, (16, 1024)), (96, (8, 480)), (512, (4, 2048))])
def test_pack_layer_other_groups(cuda, gs, shape):
    _check_pack(I.weights(*shape, seed=gs), cuda, gs)


def test_pack_layer_special_values(cuda):
    rows = [I.subnormal_block(4, 1024, seed=1), I.near_max_block(4, 1024, seed=2, amax=7e-5),
            I.near_max_block(4, 1024, seed=3, amax=3.0e38), torch.zeros(4, 1024, dtype=torch.bfloat16),
            -torch.zeros(4, 1024, dtype=torch.bfloat16), I.weights(4, 1024, seed=4, std=1e-6)]
    _check_pack(torch.cat(rows), cuda)


def test_pack_layer_every_bf16_value(cuda):
    vals = I.finite_bf16_values()
    g = I.gen(3)
    for ab in torch.randint(1, 0x7F80, (24,), generator=g).tolist() + [0x3728, 0x3727, 0x3880, 0x7F7F]:
        amax = torch.tensor([ab], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        x = vals[vals.abs() <= amax]
        x = torch.cat([x, torch.zeros((-x.numel()) % 128, dtype=torch.bfloat16)]).view(-1, 128)
        x[:, 0] = amax
        _check_pack(x, cuda)


def test_pack_layer_strided_rows(cuda):
    base = I.weights(64, 1536, seed=9)
    bg = base.to(cuda)
    for v in (lambda t: t[:, 256:1280], lambda t: t[::2], lambda t: t[:, 8:1032]):
        w, wg = v(base), v(bg)
        p, s, _ = slime_amd.pack_layer(wg, 128, True)
        po, so, _ = C.int4_pack_layer(w.contiguous(), 128, True)
        assert torch.equal(p.cpu(), po) and I.same_bits(s.cpu(), so)


@pytest.fixture(scope="module")
def vocab_ragged():
    # [151937, 2560]: N is a multiple of 128, so the reference accepts it; M is not a multiple of 8
    w = I.weights(151937, 2560, seed=11)
    w[::1000, :128] = 0
    return w


def test_pack_layer_vocab_ragged_sym(cuda, vocab_ragged):
    _check_pack(vocab_ragged, cuda)


@pytest.mark.parametrize("sym", [True, False])
def test_fake_quant_vocab_ragged(cuda, vocab_ragged, sym):
    q, s, z = slime_amd.fake_int4_quant_cuda(vocab_ragged.to(cuda), (1, 128), sym)
    assert s.shape == (151937, 20)
    qo, so, zo = C.int4_fake_quant(vocab_ragged, (1, 128), sym)
    assert I.same_bits(q.cpu(), qo) and I.same_bits(s.cpu(), so) and I.same_bits(z.cpu(), zo)


def test_pack_layer_vocab_ragged_asym(cuda, vocab_ragged):
    # asymmetric: the zero points are packed eight ROWS to a word, and 151937 rows do not divide by 8 - the
    # reference fails in zeros.reshape(-1, zeros.shape[1] // 8, 8) (convert_hf_to_int4_direct.py:137), and so does this
    with pytest.raises(RuntimeError, match="invalid for input of size"):
        slime_amd.pack_layer(vocab_ragged.to(cuda), 128, False)
    # the largest multiple of 8 rows goes through, bit for bit
    w = vocab_ragged[:151936]
    p, s, z = slime_amd.pack_layer(w.to(cuda), 128, False)
    po, so, zo = C.int4_pack_layer(w, 128, False)
    assert torch.equal(p.cpu(), po) and I.same_bits(s.cpu(), so) and torch.equal(z.cpu(), zo)


def test_pack_layer_ragged_n_fails_like_reference(cuda):
    w = I.weights(4100, 3000, seed=1).to(cuda)
    with pytest.raises(RuntimeError):
        slime_amd.pack_layer(w, 128, True)      # the reference fails in .view(M, 1, N // 128, 128)


@pytest.mark.parametrize("block", [(1, 32), (1, 128), (1, 64), (32, 1), (4, 8), (2, 16), (1, 256)])
@pytest.mark.parametrize("sym", [True, False])
def test_fake_quant(cuda, block, sym):
    w = I.weights(70, 300, seed=block[0] * 100 + block[1])
    for x in (w, w.float(), w.t()):
        q, s, z = slime_amd.fake_int4_quant_cuda(x.to(cuda), block, sym)
        assert q.dtype == x.dtype and s.dtype == x.dtype and z.dtype == x.dtype
        qo, so, zo = C.int4_fake_quant(x, block, sym)
        assert I.same_bits(q.cpu(), qo) and I.same_bits(s.cpu(), so) and I.same_bits(z.cpu(), zo)


def _fake_quant_same(q, s, z, qo, so, zo):
    nan = qo.isnan()
    assert torch.equal(q.isnan(), nan) and torch.equal(q[~nan].view(torch.int16), qo[~nan].view(torch.int16))
    assert I.same_bits(s, so) and I.same_bits(z, zo)


@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("sym", [True, False])
def test_fake_quant_row_groups_fast_layout(cuda, gs, sym):
    # contiguous-row bf16 with groups that tile the row: the layout pack_layer and the QAT callers use
    w = I.weights(333, 1024, seed=gs, outlier_p=0.01)
    w[0, :gs] = 0
    w[1, :gs] = -0.0
    w[2, :256] = I.subnormal_block(1, 256, seed=1)[0]
    w[3, :256] = I.near_max_block(1, 256, seed=2, amax=3.0e38)[0]
    w[4, :256] = I.weights(1, 256, seed=4, std=1e-6)[0]
    wg = w.to(cuda)
    for view in (lambda t: t, lambda t: t[:, 128:896], lambda t: t[::3], lambda t: t[5:, 256:]):
        q, s, z = slime_amd.fake_int4_quant_cuda(view(wg), (1, gs), sym)
        _fake_quant_same(q.cpu(), s.cpu(), z.cpu(), *C.int4_fake_quant(view(w), (1, gs), sym))
    bad = w.clone()
    bad[7, 5] = float("nan")
    bad[8, 130] = float("inf")
    bad[9, :gs] = float("nan")
    q, s, z = slime_amd.fake_int4_quant_cuda(bad.to(cuda), (1, gs), sym)
    qo, so, zo = C.int4_fake_quant(bad, (1, gs), sym)
    ok = torch.ones(333, dtype=torch.bool)
    ok[7:10] = False                                 # rows with NaN / Inf: only NaN-ness of the codes is specified
    _fake_quant_same(q.cpu()[ok], s.cpu()[ok], z.cpu()[ok], qo[ok], so[ok], zo[ok])
    assert torch.equal(q.cpu()[~ok].isnan(), qo[~ok].isnan())


@pytest.mark.parametrize("sym", [True, False])
def test_fake_quant_every_bf16_value(cuda, sym):
    vals = I.finite_bf16_values()
    g = I.gen(13)
    rows = []
    for ab in torch.randint(1, 0x7F80, (16,), generator=g).tolist() + [0x3728, 0x3727, 0x7F7F, 1]:
        amax = torch.tensor([ab], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        x = vals[vals.abs() <= amax]
        x = torch.cat([x, torch.zeros((-x.numel()) % 1024, dtype=torch.bfloat16)]).view(-1, 128)
        x[:, 0] = amax
        rows.append(x.reshape(-1, 1024))
    w = torch.cat(rows)
    q, s, z = slime_amd.fake_int4_quant_cuda(w.to(cuda), (1, 128), sym)
    _fake_quant_same(q.cpu(), s.cpu(), z.cpu(), *C.int4_fake_quant(w, (1, 128), sym))


def test_fake_quant_asym_many_scales(cuda):
    # the asymmetric quotients use a reciprocal and a two-FMA correction: 4M elements under ~32k different scales,
    # with offsets (one-sided groups), tiny ranges (1e-5 floor) and ties (bf16 data makes x / scale land on .5 often)
    g = I.gen(77)
    base = torch.randn(4096, 1024, generator=g)
    scale = torch.exp(torch.empty(4096, 8, 1).uniform_(-12.0, 6.0, generator=g))
    shift = torch.randn(4096, 8, 1, generator=g) * (torch.rand(4096, 8, 1, generator=g) < 0.3)
    w = ((base.view(4096, 8, 128) + shift) * scale).view(4096, 1024).to(torch.bfloat16)
    q, s, z = slime_amd.fake_int4_quant_cuda(w.to(cuda), (1, 128), False)
    _fake_quant_same(q.cpu(), s.cpu(), z.cpu(), *C.int4_fake_quant(w, (1, 128), False))
    w8 = w[:, :512].contiguous()
    p, sc, pz = slime_amd.pack_layer(w8.to(cuda), 128, False)
    po, so, pzo = C.int4_pack_layer(w8, 128, False)
    assert torch.equal(p.cpu(), po) and I.same_bits(sc.cpu(), so) and torch.equal(pz.cpu(), pzo)


def test_fake_quant_ragged_big(cuda):
    w = I.weights(4100, 3000, seed=2)
    q, s, z = slime_amd.fake_int4_quant_cuda(w.to(cuda), (1, 128), True)
    qo, so, zo = C.int4_fake_quant(w, (1, 128), True)
    assert s.shape == (4100, 24)
    assert I.same_bits(q.cpu(), qo) and I.same_bits(s.cpu(), so) and I.same_bits(z.cpu(), zo)


def test_fake_quant_errors(cuda):
    w = torch.zeros(64, 64, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(RuntimeError, match="divisible by 32"):
        slime_amd.fake_int4_quant_cuda(w, (1, 48), True)
    with pytest.raises(RuntimeError, match="2D"):
        slime_amd.fake_int4_quant_cuda(w.view(-1), (1, 32), True)
    with pytest.raises(RuntimeError, match="not supported"):
        slime_amd.fake_int4_quant_cuda(w, (2, 64), True)
    with pytest.raises(RuntimeError, match="positive"):
        slime_amd.fake_int4_quant_cuda(w, (0, 32), True)


@pytest.mark.parametrize("shape,gs", [((16, 256), 128), ((8, 2048), 128), ((24, 96), 32)])
def test_pack_layer_asym(cuda, shape, gs):
    w = I.weights(*shape, seed=shape[1])
    p, s, z = slime_amd.pack_layer(w.to(cuda), gs, False)
    po, so, zo = C.int4_pack_layer(w, gs, False)
    assert torch.equal(p.cpu(), po) and I.same_bits(s.cpu(), so) and torch.equal(z.cpu(), zo)


def _check_pack_asym(w, cuda, gs=128, view=None):
    wg = w.to(cuda)
    if view is not None:
        wg, w = view(wg), view(w).contiguous()
    p, s, z = slime_amd.pack_layer(wg, gs, False)
    po, so, zo = C.int4_pack_layer(w, gs, False)
    nbad = int((p.cpu() != po).sum())
    assert nbad == 0, f"{nbad} packed-word mismatches"
    assert I.same_bits(s.cpu(), so) and torch.equal(z.cpu(), zo)


@pytest.mark.parametrize("shape,gs", [((768, 2048), 128), ((2048, 768), 128), ((40, 7168), 128), ((64, 96), 32),
                                      ((336, 1024), 64), ((1000, 2560), 128)])
def test_pack_layer_asym_fused(cuda, shape, gs):
    w = I.weights(*shape, seed=shape[1] + 1, outlier_p=0.01)
    w[0, :gs] = 0
    _check_pack_asym(w, cuda, gs)


def test_pack_layer_asym_one_sided_groups_and_extremes(cuda):
    # all-positive / all-negative groups give codes far above 15 (the reference packs them unmasked), huge values
    # give scales where the dequantise / re-quantise chain is not the identity, tiny ones hit the 1e-5 floor
    rows = [I.weights(8, 1024, seed=1).abs() + 0.5, -(I.weights(8, 1024, seed=2).abs()) - 0.25,
            I.near_max_block(8, 1024, seed=3, amax=3.0e38), I.near_max_block(8, 1024, seed=4, amax=1.0e37).abs(),
            I.subnormal_block(8, 1024, seed=5), I.weights(8, 1024, seed=6, std=1e-6),
            torch.zeros(8, 1024, dtype=torch.bfloat16), -torch.zeros(8, 1024, dtype=torch.bfloat16),
            I.weights(8, 1024, seed=7) + 3.0]
    _check_pack_asym(torch.cat(rows), cuda)


def test_pack_layer_asym_every_bf16_value(cuda):
    vals = I.finite_bf16_values()
    g = I.gen(23)
    rows = []
    for ab in torch.randint(0x3000, 0x7F80, (12,), generator=g).tolist() + [0x3728, 0x7F7F, 0x7C80]:
        amax = torch.tensor([ab], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        x = vals[vals.abs() <= amax]
        x = torch.cat([x, torch.zeros((-x.numel()) % 1024, dtype=torch.bfloat16)]).view(-1, 128)
        x[:, 0] = amax
        x[:, 1] = -amax
        rows.append(x.reshape(-1, 1024))
    w = torch.cat(rows)
    w = w[: w.shape[0] // 8 * 8]
    _check_pack_asym(w, cuda)


def test_pack_layer_asym_strided_rows(cuda):
    w = I.weights(64, 1536, seed=9)
    _check_pack_asym(w, cuda, 128, view=lambda t: t[:, 256:1280])
    _check_pack_asym(w, cuda, 128, view=lambda t: t[::2])


def test_pack_plan_moe_experts(cuda):
    # Qwen3-30B-A3B expert shapes: 8 experts x {gate, up [768,2048], down [2048,768]} in one launch
    ws = []
    for e in range(8):
        ws += [I.weights(768, 2048, seed=3 * e), I.weights(768, 2048, seed=3 * e + 1), I.weights(2048, 768, seed=3 * e + 2)]
    plan = slime_amd.Int4PackPlan([w.to(cuda) for w in ws], 128)
    for w, (p, s) in zip(ws, plan.run()):
        po, so, _ = C.int4_pack_layer(w, 128, True)
        assert torch.equal(p.cpu(), po) and I.same_bits(s.cpu(), so)
    # reconstruction error bound: |w - (nib-8)*scale| <= scale/2 (+ bf16 rounding of the scale)
    p, s = plan.outputs[0]
    nib = torch.stack([(p >> (4 * j)) & 0xF for j in range(8)], dim=-1).view(768, 2048).float() - 8
    sf = s.float().repeat_interleave(128, dim=1)
    assert ((nib * sf - ws[0].to(cuda).float()).abs() <= sf * (0.5 + 7 * 2 ** -8)).all()


def test_pack_plan_many_small_tensors_uses_item_table(cuda):
    # 24 tensors keep the searched launch (above); 90 mixed tensors get one pre-resolved descriptor per work item
    shapes = [(96, 256), (33, 768), (1, 128), (64, 128), (7, 7168), (128, 2048), (5, 384), (200, 1024), (63, 128)] * 10
    ws = [I.weights(*sh, seed=200 + i) for i, sh in enumerate(shapes)]
    plan = slime_amd.Int4PackPlan([w.to(cuda) for w in ws], 128)
    assert plan._items is not None and plan._items.shape == (plan.total_work, 4)
    for w, (p, s) in zip(ws, plan.run()):
        po, so, _ = C.int4_pack_layer(w, 128, True)
        assert torch.equal(p.cpu(), po) and I.same_bits(s.cpu(), so)
    plan32 = slime_amd.Int4PackPlan([w.to(cuda) for w in ws[:70]], 32)
    for w, (p, s) in zip(ws, plan32.run()):
        po, so, _ = C.int4_pack_layer(w, 32, True)
        assert torch.equal(p.cpu(), po) and I.same_bits(s.cpu(), so)


def test_int4_golden(cuda):
    from safetensors.torch import load_file

    f = load_file(os.path.join(GOLDEN, "int4_golden.safetensors"))
    for case in sorted({k.split("/")[0] for k in f}):
        w = f[f"{case}/w"].to(cuda)
        gs = int(case.split("_")[0][1:])
        q, s, _ = slime_amd.fake_int4_quant_cuda(w, (1, gs), True)
        assert I.same_bits(q.cpu(), f[f"{case}/q"]) and I.same_bits(s.cpu(), f[f"{case}/scale"]), case
        p, s2, _ = slime_amd.pack_layer(w, gs, True)
        assert torch.equal(p.cpu(), f[f"{case}/packed"]) and I.same_bits(s2.cpu(), f[f"{case}/pack_scale"]), case
        d = slime_amd.dequantize_int4(p, s2, torch.tensor(list(w.shape)), gs)
        assert I.same_bits(d.cpu(), f[f"{case}/deq"]), case
        for arith, tag in (("cpu", "ste"), ("device", "ste_dev")):
            with slime_amd.torch_arithmetic(arith):
                assert I.same_bits(slime_amd.fake_int4_quantization_ste(w, gs).cpu(), f[f"{case}/{tag}"]), (case, arith)
        if f"{case}/packed_asym" in f:
            pa, _, pz = slime_amd.pack_layer(w, gs, False)
            assert torch.equal(pa.cpu(), f[f"{case}/packed_asym"]) and torch.equal(pz.cpu(), f[f"{case}/packed_zp"])


def test_pack_helpers_on_gpu(cuda):
    g = I.gen(0)
    q = torch.randint(-8, 8, (9, 37), generator=g, dtype=torch.int32).to(torch.int8)
    from oracle import torch_ref as T

    assert torch.equal(slime_amd.pack_to_int32(q.to(cuda), 4, sym=True).cpu(), T.pack_to_int32_ref(q, 4, sym=True))
    with pytest.raises(ValueError):
        slime_amd.pack_to_int32(q.to(cuda), 9)
    x = I.weights(8, 256, seed=1)
    sc = (x.float().abs().view(8, 2, 128).amax(-1) / 7).to(torch.bfloat16)
    assert torch.equal(slime_amd.quantize(x.to(cuda), sc.to(cuda), None).cpu(), T.quantize_ref(x, sc, None))


# ------------------------------------------------------------------ INT4 -> bf16

def _same_or_both_nan(a, b):
    nan = b.isnan()
    return torch.equal(a.isnan(), nan) and torch.equal(a[~nan].view(torch.int16), b[~nan].view(torch.int16))


@pytest.mark.parametrize("shape,gs", [((768, 2048), 128), ((2048, 768), 128), ((16, 256), 128), ((33, 768), 128),
                                      ((1, 128), 128), ((7, 7168), 128), ((24, 96), 32), ((333, 1024), 64),
                                      ((5, 40), 8), ((3, 96), 48), ((1000, 2560), 128)])
def test_int4_dequant(cuda, shape, gs):
    g = I.gen(shape[0] + gs)
    packed = torch.randint(-2 ** 31, 2 ** 31, (shape[0], shape[1] // 8), generator=g, dtype=torch.int64).to(torch.int32)
    scale = (I.log_uniform_scales(shape[0], shape[1] // gs, seed=gs) * 0.1).to(torch.bfloat16)
    got = slime_amd.dequantize_int4(packed.to(cuda), scale.to(cuda), shape, gs)
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == shape and got.is_contiguous()
    assert I.same_bits(got.cpu(), C.int4_dequant(packed, scale, shape, gs))


def test_int4_dequant_every_nibble_times_every_scale(cuda):
    # 16 nibble values x all 65536 bf16 scale bit patterns (NaN scales: NaN-ness only)
    scale = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).view(-1, 1)
    word = sum(((j * 2 + 1) % 16) << (4 * j) for j in range(8))          # nibbles 1,3,..,15
    word2 = sum(((j * 2) % 16) << (4 * j) for j in range(8))              # nibbles 0,2,..,14
    packed = torch.tensor([word, word2], dtype=torch.int64).to(torch.int32).repeat(65536, 1)
    got = slime_amd.dequantize_int4(packed.to(cuda), scale.to(cuda), (65536, 16), 16).cpu()
    assert _same_or_both_nan(got, C.int4_dequant(packed, scale, (65536, 16), 16))


def test_int4_dequant_inverts_pack_layer(cuda):
    w = I.weights(768, 2048, seed=12)
    p, s, _ = slime_amd.pack_layer(w.to(cuda), 128, True)
    d = slime_amd.dequantize_int4(p, s, (768, 2048), 128)
    assert I.same_bits(d.cpu(), C.int4_dequant(*C.int4_pack_layer(w, 128, True)[:2], (768, 2048), 128))
    # a second pack of the dequantised weight reproduces the words wherever the group's largest code was +-7
    step = s.float().repeat_interleave(128, 1)
    assert ((d.float() - w.to(cuda).float()).abs() <= step * (0.5 + 7 * 2.0 ** -8) + d.float().abs() * 2.0 ** -8).all()


def test_int4_dequant_errors(cuda):
    p = torch.zeros(4, 16, dtype=torch.int32, device=cuda)
    s = torch.ones(4, 1, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(ValueError):
        slime_amd.dequantize_int4(p, s, (4, 128), 100)
    with pytest.raises(ValueError):
        slime_amd.dequantize_int4(p, s, (4, 256), 128)
    with pytest.raises(ValueError, match="incompatible"):
        slime_amd.dequantize_int4(p, s.repeat(1, 2), (4, 128), 128)
    with pytest.raises(RuntimeError):
        slime_amd.dequantize_int4(p.cpu(), s.cpu(), (4, 128), 128)


# ------------------------------------------------------------------ QAT straight-through forward

ARITH = {0: "cpu", 1: "device"}


@pytest.mark.parametrize("shape,gs", [((768, 2048), 128), ((16, 256), 128), ((33, 768), 128), ((1, 128), 128),
                                      ((7, 7168), 128), ((24, 96), 32), ((333, 1024), 64), ((1000, 2560), 128)])
def test_fake_ste_forward(cuda, shape, gs):
    w = I.weights(*shape, seed=shape[1] + gs, outlier_p=0.01)
    w[0, :gs] = 0
    for div7, arith in ARITH.items():
        with slime_amd.torch_arithmetic(arith):
            y = slime_amd.fake_int4_quantization_ste(w.to(cuda), gs)
        assert y.dtype == torch.bfloat16 and y.shape == w.shape
        assert I.same_bits(y.cpu(), C.int4_fake_ste(w, gs, div7)), arith


def test_fake_ste_special_values_and_every_bf16_value(cuda):
    rows = [I.subnormal_block(4, 1024, seed=1), I.near_max_block(4, 1024, seed=2, amax=7e-5),
            I.near_max_block(4, 1024, seed=3, amax=3.0e38), torch.zeros(4, 1024, dtype=torch.bfloat16),
            -torch.zeros(4, 1024, dtype=torch.bfloat16), I.weights(4, 1024, seed=4, std=1e-6)]
    vals = I.finite_bf16_values()
    g = I.gen(3)
    for ab in torch.randint(1, 0x7F80, (12,), generator=g).tolist() + [0x3728, 0x3727, 0x7F7F]:
        amax = torch.tensor([ab], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        x = vals[vals.abs() <= amax]
        x = torch.cat([x, torch.zeros((-x.numel()) % 1024, dtype=torch.bfloat16)]).view(-1, 128)
        x[:, 0] = amax
        rows.append(x.reshape(-1, 1024))
    w = torch.cat(rows)
    nan_row = I.weights(2, 1024, seed=9)
    nan_row[0, 5] = float("nan")
    nan_row[1, 300] = float("inf")
    w = torch.cat([w, nan_row])
    for div7, arith in ARITH.items():
        with slime_amd.torch_arithmetic(arith):
            y = slime_amd.fake_int4_quantization_ste(w.to(cuda), 128).cpu()
        assert _same_or_both_nan(y, C.int4_fake_ste(w, 128, div7)), arith


def test_fake_ste_matches_torch_ops_on_the_gpu(cuda):
    # the reference's own op sequence executed by torch on the GPU, against the kernel ("device" arithmetic)
    from oracle import torch_ref as T

    for shape, gs in (((512, 2048), 128), ((64, 96), 32), ((100, 1024), 64)):
        w = I.weights(*shape, seed=shape[0], outlier_p=0.01).to(cuda)
        assert I.same_bits(slime_amd.fake_int4_quantization_ste(w, gs).cpu(), T.fake_int4_ste_ref(w, gs).cpu())


def test_fake_ste_ragged_and_gradient(cuda):
    from oracle import torch_ref as T

    w = I.weights(6, 100, seed=3)
    for div7, arith in ARITH.items():
        with slime_amd.torch_arithmetic(arith):
            y = slime_amd.fake_int4_quantization_ste(w.to(cuda), 64)          # N % group != 0: zero-padded groups
        assert I.same_bits(y.cpu(), T.fake_int4_ste_ref(w, 64, device_arith=bool(div7))), arith
    x = I.weights(16, 256, seed=4).to(cuda).requires_grad_(True)
    x.main_grad = torch.zeros(16, 256, device=cuda)
    y = slime_amd.fake_int4_quantization_ste(x, 128)
    assert y.main_grad is x.main_grad
    gy = torch.randn(16, 256, device=cuda).to(torch.bfloat16)
    y.backward(gy)
    assert torch.equal(x.grad, gy)                                            # straight-through: identity


def test_grouped_search_entry_point(cuda):
    # Int4PackPlan uses the per-item table; the descriptor-array + prefix-sum form stays part of the C ABI
    from slime_amd import _lib

    shapes = [(768, 2048), (33, 768), (1, 128), (2048, 768), (7, 7168)]
    ws = [I.weights(*sh, seed=50 + i) for i, sh in enumerate(shapes)]
    wg = [w.to(cuda) for w in ws]
    outs, rows, starts, work = [], [], [0], 0
    for w in wg:
        M, N = w.shape
        p = torch.empty(M, N // 8, dtype=torch.int32, device=cuda)
        sc = torch.empty(M, N // 128, dtype=torch.bfloat16, device=cuda)
        outs.append((p, sc))
        rows.append([w.data_ptr(), p.data_ptr(), sc.data_ptr(), M * N // 128])
        work += -(-(M * N // 128) // _lib.INT4_GROUPS_PER_WG)
        starts.append(work)
    descs = torch.tensor(rows, dtype=torch.int64).to(cuda)
    st = torch.tensor(starts, dtype=torch.int64).to(cuda)
    rc = _lib.load().wq_int4_group_quant_pack_grouped(descs.data_ptr(), st.data_ptr(), len(ws), work, 128,
                                                      _lib.stream_ptr(cuda))
    _lib.check(rc, "grouped")
    for w, (p, sc) in zip(ws, outs):
        po, so, _ = C.int4_pack_layer(w, 128, True)
        assert torch.equal(p.cpu(), po) and I.same_bits(sc.cpu(), so)


def test_fake_ste_many_scales_both_rules(cuda):
    g = I.gen(78)
    base = torch.randn(4096, 1024, generator=g)
    scale = torch.exp(torch.empty(4096, 8, 1).uniform_(-12.0, 6.0, generator=g))
    w = (base.view(4096, 8, 128) * scale).view(4096, 1024).to(torch.bfloat16)
    for div7, arith in ARITH.items():
        with slime_amd.torch_arithmetic(arith):
            y = slime_amd.fake_int4_quantization_ste(w.to(cuda), 128)
        assert I.same_bits(y.cpu(), C.int4_fake_ste(w, 128, div7)), arith


def test_int4_dequant_plan(cuda):
    shapes = [(96, 256), (33, 768), (1, 128), (64, 128), (7, 7168), (128, 2048), (5, 384), (200, 1024), (63, 128), (768, 2048)]
    for gs in (128, 32):
        trip = [C.int4_pack_layer(I.weights(*sh, seed=400 + i), gs, True)[:2] for i, sh in enumerate(shapes)]
        plan = slime_amd.Int4DequantPlan([p.to(cuda) for p, _ in trip], [s.to(cuda) for _, s in trip],
                                         [torch.tensor(sh) for sh in shapes], gs)
        for (p, s), sh, y in zip(trip, shapes, plan.run()):
            assert tuple(y.shape) == sh and I.same_bits(y.cpu(), C.int4_dequant(p, s, sh, gs))
    with pytest.raises(ValueError):
        slime_amd.Int4DequantPlan([trip[0][0].to(cuda)], [trip[0][1].to(cuda)], [shapes[0]], 96)
    with pytest.raises(ValueError):
        slime_amd.Int4DequantPlan([trip[0][0].to(cuda)], [trip[0][1].to(cuda)], [(96, 512)], 32)


@pytest.mark.parametrize("group", [128, 64, 32])
def test_bucket_form_with_destinations_at_every_word_offset_of_a_line(cuda, group):
    """A bucket packs its outputs back to back, so the packed words of a tensor start wherever the previous tensor
    ended.  Items whose words do not start on a 128-byte line are collected in LDS and written out as whole lines:
    every 4-byte offset inside a line, with full, short and one-group items, against the oracle - and the bytes around
    every output must stay untouched."""
    from slime_amd import _lib
    from slime_amd.int4 import item_table

    shapes = [(64, 128), (1, 128), (63, 128), (65, 128), (3, 1024), (130, 256), (16, 2048), (7, 384)]
    ws = [I.weights(*sh, seed=900 + i) for i, sh in enumerate(shapes)]
    wg = [w.to(cuda) for w in ws]
    for shift in range(0, 128, 4):
        rows, places, off = [], [], 128 + shift
        for w in wg:
            M, N = w.shape
            p0 = off
            s0 = p0 + M * N // 2
            off = -(-(s0 + M * N // group * 2) // 4) * 4 + 8   # the weight_shape entry of a bucket: the next tensor lands 8 bytes further
            rows.append([w.data_ptr(), p0, s0, M * N // group])
            places.append((p0, s0, M, N))
        table, _, _ = item_table(rows, group)
        out = torch.full((off + 256,), 0xA5, dtype=torch.uint8, device=cuda)
        rc = _lib.load().wq_int4_bucket_convert(table.contiguous().to(cuda).data_ptr(), table.shape[0], out.data_ptr(), group,
                                                _lib.stream_ptr(cuda))
        _lib.check(rc, "bucket form")
        host = out.cpu()
        written = torch.zeros(host.numel(), dtype=torch.bool)
        for w, (p0, s0, M, N) in zip(ws, places):
            po, so, _ = C.int4_pack_layer(w, group, True)
            assert torch.equal(host[p0:p0 + M * N // 2].clone().view(torch.int32).view(M, N // 8), po), (shift, M, N)
            assert torch.equal(host[s0:s0 + M * N // group * 2].clone().view(torch.int16), so.view(torch.int16).reshape(-1)), (shift, M, N)
            written[p0:s0 + M * N // group * 2] = True
        assert bool((host[~written] == 0xA5).all()), shift


def test_asym_bucket_form_with_destinations_off_a_line(cuda):
    """The asymmetric items kernel with packed words starting at every fourth word offset of a 128-byte line."""
    from slime_amd import _lib
    from slime_amd.int4 import item_table

    group = 128
    shapes = [(64, 128), (8, 128), (72, 256), (16, 2048), (136, 384)]
    ws = [I.weights(*sh, seed=950 + i) + 0.01 for i, sh in enumerate(shapes)]
    wg = [w.to(cuda) for w in ws]
    for shift in range(0, 128, 16):
        rows, places, off, zoff = [], [], 128 + shift + 4, 0
        for w in wg:
            M, N = w.shape
            p0 = off
            s0 = p0 + M * N // 2
            off = -(-(s0 + M * N // group * 2) // 4) * 4 + 8
            rows.append([w.data_ptr(), p0, s0, zoff, M * N // group])
            places.append((p0, s0, zoff, M, N))
            zoff += (2 * M * N // group + 15) // 16 * 16
        full = torch.tensor(rows, dtype=torch.int64)
        table4, owner, local = item_table(full[:, [0, 1, 2, 4]], group)
        zcol = full[owner, 3] + local * (_lib.INT4_GROUPS_PER_WG * 2)
        table = torch.cat([table4[:, :3], zcol.unsqueeze(1), table4[:, 3:]], dim=1).contiguous().to(cuda)
        out = torch.full((off + 256,), 0x5A, dtype=torch.uint8, device=cuda)
        zero = torch.zeros(zoff + 16, dtype=torch.uint8, device=cuda)
        rc = _lib.load().wq_int4_group_quant_pack_asym_items(table.data_ptr(), table.shape[0], out.data_ptr(), zero.data_ptr(),
                                                             group, _lib.stream_ptr(cuda))
        _lib.check(rc, "asym items")
        host, zhost = out.cpu(), zero.cpu()
        written = torch.zeros(host.numel(), dtype=torch.bool)
        for w, (p0, s0, z0, M, N) in zip(ws, places):
            po, so, _ = C.int4_pack_layer(w, group, False)
            _, _, zo = C.int4_fake_quant(w, (1, group), False)
            assert torch.equal(host[p0:p0 + M * N // 2].clone().view(torch.int32).view(M, N // 8), po), (shift, M, N)
            assert torch.equal(host[s0:s0 + M * N // group * 2].clone().view(torch.int16), so.view(torch.int16).reshape(-1)), (shift, M, N)
            assert torch.equal(zhost[z0:z0 + M * N // group * 2].clone().view(torch.int16), zo.view(torch.int16).reshape(-1)), (shift, M, N)
            written[p0:s0 + M * N // group * 2] = True
        assert bool((host[~written] == 0x5A).all()), shift
