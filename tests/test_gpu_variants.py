"""The adjacent format variants on the GPU, against the CPU oracle: power-of-two (UE8M0) block scales, fp64 input to
the fake-INT4 quantiser, INT4 -> bf16 with fp16 / fp32 / per-element scales and ragged rows."""

import pytest
import torch

import slime_amd
from oracle import c_oracle as C
from slime_amd import processors
from tests import wq_inputs as I

pytestmark = pytest.mark.gpu
E4M3 = torch.float8_e4m3fn


@pytest.mark.parametrize("shape", [(128, 128), (256, 384), (300, 200), (7, 7168), (129, 127), (4100, 3000), (1024, 2560)])
def test_ue8m0_block_quant_matches_oracle(cuda, shape):
    # PARITY UNPINNED against sglang's quant_weight_ue8m0 (not vendored); bit-exact against this build's restatement
    w = I.zero_blocks(I.weights(*shape, seed=sum(shape)), 0.2, seed=1)
    q, s = slime_amd.quant_weight_ue8m0(w.to(cuda), [128, 128])
    qo, so = C.fp8_block_quant(w, (128, 128), 3)
    assert q.dtype == E4M3 and s.dtype == torch.float32
    assert torch.equal(q.cpu().view(torch.uint8), qo) and torch.equal(s.cpu().view(torch.int32), so.view(torch.int32))
    mant, _ = torch.frexp(s.cpu().double())
    assert (mant == 0.5).all()


def test_ue8m0_every_bf16_value_and_views(cuda):
    vals = I.finite_bf16_values()
    g = I.gen(31)
    for ab in torch.randint(1, 0x7F80, (24,), generator=g).tolist() + [0x3F60, 0x38D1, 0x38D2, 0x7F7F, 1]:
        amax = torch.tensor([ab], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        x = vals[vals.abs() <= amax]
        x = torch.cat([x, torch.zeros((-x.numel()) % (128 * 128), dtype=torch.bfloat16)]).view(-1, 128)
        x[::128, 0] = amax
        q, s = slime_amd.quant_weight_ue8m0(x.to(cuda), [128, 128])
        qo, so = C.fp8_block_quant(x, (128, 128), 3)
        assert torch.equal(q.cpu().view(torch.uint8), qo) and torch.equal(s.cpu().view(torch.int32), so.view(torch.int32)), ab
    base = I.weights(512, 776, seed=4)
    for v in (lambda t: t[:, 128:640], lambda t: t.t(), lambda t: t[::2, ::3], lambda t: t[:, 1:769]):
        from slime_amd import _lib, fp8
        q, s = fp8._block_quant(v(base.to(cuda)), 128, 128, _lib.FP8_MODE_UE8M0, "t")
        qo, so = C.fp8_block_quant(v(base), (128, 128), 3)
        assert torch.equal(q.cpu().view(torch.uint8), qo) and torch.equal(s.cpu().view(torch.int32), so.view(torch.int32))
    bad = I.weights(128, 256, seed=6)
    bad[3, 3] = float("nan")
    bad[5, 130] = float("inf")
    q, s = slime_amd.quant_weight_ue8m0(bad.to(cuda), [128, 128])
    qo, so = C.fp8_block_quant(bad, (128, 128), 3)
    assert s[0, 0].isnan() and s[0, 1].isinf()
    assert torch.equal((q.cpu().view(torch.uint8) & 0x7F) == 0x7F, (qo & 0x7F) == 0x7F)
    with pytest.raises(TypeError):
        slime_amd.quant_weight_ue8m0(bad.float().to(cuda), [128, 128])


def test_quantize_param_ue8m0_branch(cuda):
    w = I.weights(256, 384, seed=9).to(cuda)
    name = "model.layers.0.mlp.down_proj.weight"
    try:
        processors.set_ue8m0_requant(True)
        with pytest.raises(NotImplementedError):          # the DeepGEMM scale layout is not produced: refused, not ignored
            slime_amd._quantize_param(name, w, [128, 128], transform_ue8m0=True)
        (n0, q), (n1, s) = slime_amd._quantize_param(name, w, [128, 128], transform_ue8m0=False)
        qo, so = C.fp8_block_quant(w.cpu(), (128, 128), 3)
        assert n0 == name and n1 == "model.layers.0.mlp.down_proj.weight_scale_inv"
        assert torch.equal(q.cpu().view(torch.uint8), qo) and torch.equal(s.cpu().view(torch.int32), so.view(torch.int32))
        cfg = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic", "weight_block_size": [128, 128]}
        mn = "module.module.decoder.layers.0.mlp.linear_fc1.weight"
        out = slime_amd.quantize_params_fp8(None, mn, [("a.gate_proj.weight", w), ("a.up_proj.weight", w)], cfg, transform_ue8m0=False)
        assert torch.equal(out[1][1].cpu().view(torch.int32), so.view(torch.int32))
        from slime_amd import bucket as B
        got = B.BucketConverter(None, cfg, transform_ue8m0=False).convert([(mn, [("a.gate_proj.weight", w)])])
        assert torch.equal(dict(got.reconstruct_tensors())["a.gate_proj.weight_scale_inv"].cpu().view(torch.int32), so.view(torch.int32))
    finally:
        processors.set_ue8m0_requant(False)
    (_, q), (_, s) = slime_amd._quantize_param(name, w, [128, 128], transform_ue8m0=True)       # switch off: flag has no effect
    qo, so = C.fp8_block_quant(w.cpu(), (128, 128), 1)
    assert torch.equal(q.cpu().view(torch.uint8), qo) and torch.equal(s.cpu().view(torch.int32), so.view(torch.int32))


@pytest.mark.parametrize("sym", [True, False])
@pytest.mark.parametrize("block", [(1, 128), (1, 32), (32, 1), (4, 8)])
def test_fake_quant_fp64(cuda, sym, block):
    g = I.gen(block[0] + block[1])
    x = torch.randn(70, 300, generator=g, dtype=torch.float64) * 0.02
    for view in (lambda t: t, lambda t: t.t()):
        q, s, z = slime_amd.fake_int4_quant_cuda(view(x.to(cuda)), block, sym)
        qo, so, zo = C.int4_fake_quant(view(x), block, sym)
        assert q.dtype == torch.float64 and s.dtype == torch.float64
        assert torch.equal(q.cpu(), qo) and torch.equal(s.cpu(), so) and torch.equal(z.cpu(), zo)
    with pytest.raises(RuntimeError, match="not implemented for 'Half'"):
        slime_amd.fake_int4_quant_cuda(x.half().to(cuda), block, sym)


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16, torch.float32, torch.float64])
@pytest.mark.parametrize("gs,shape", [(128, (33, 768)), (32, (24, 96)), (24, (8, 96)), (-1, (9, 52)), (1, (5, 64)), (64, (300, 1024))])
def test_dequantize_int4_any_scale_dtype(cuda, dt, gs, shape):
    g = I.gen(gs + shape[1])
    M, N = shape
    group = gs if gs > 0 else 1
    packed = torch.randint(-2 ** 31, 2 ** 31 - 1, (M, -(-N // 8)), generator=g, dtype=torch.int64).to(torch.int32)
    scale = (torch.rand(M, N // group, generator=g, dtype=torch.float64) * 0.02 + 1e-4).to(dt)
    got = slime_amd.dequantize_int4(packed.to(cuda), scale.to(cuda), torch.tensor([M, N]), gs)
    sc = scale.float() if dt == torch.float64 else scale          # the reference converts with .to(float32)
    want = C.int4_dequant_any(packed, sc, (M, N), gs)
    assert got.dtype == torch.bfloat16 and I.same_bits(got.cpu(), want)
    if dt == torch.bfloat16 and gs == 128:
        flat = slime_amd.dequantize_int4(packed.to(cuda), scale.view(-1).to(cuda), (M, N), gs) if N == 128 else None
        assert flat is None or I.same_bits(flat.cpu(), want)
    with pytest.raises(ValueError, match="incompatible"):
        slime_amd.dequantize_int4(packed.to(cuda), scale[:, :-1].to(cuda) if scale.shape[1] > 1 else scale[:-1].to(cuda), (M, N), gs)
