"""The BASELINE configurations at their full sizes.  The CPU oracle cannot cover tens of gigabytes, so these
tests combine (a) the oracle on sampled stripes of the very tensors that were processed (blocks, row groups and
row stripes are independent, so a stripe of the output depends on the same stripe of the input only), (b) equality
of the one-launch bucket results with per-tensor calls, compared on the GPU, and (c) size-independent properties:
reconstruction error bounds and encode -> decode round trips."""

import pytest
import torch

import slime_amd
from oracle import c_oracle as C

pytestmark = pytest.mark.gpu
E4M3 = torch.float8_e4m3fn

QWEN3_4B_LAYER = [(4096, 2560), (1024, 2560), (1024, 2560), (2560, 4096), (9728, 2560), (9728, 2560), (2560, 9728)]


def _gen(shape, dev, g, outliers):
    w = torch.empty(shape, dtype=torch.bfloat16, device=dev).normal_(0.0, 0.02, generator=g)
    if outliers:
        w[torch.rand(shape, device=dev, generator=g) < 1e-3] *= 20
    return w


def _stripe_rows(M, g, n=3):
    tops = torch.randint(0, max(M // 128, 1), (n,), generator=g).tolist()
    return sorted({t * 128 for t in tops} | {(M - 1) // 128 * 128})


def test_qwen3_4b_state_dict_block_fp8(cuda):
    g = torch.Generator(device=cuda).manual_seed(0)
    cg = torch.Generator().manual_seed(0)
    ws = [_gen(sh, cuda, g, False) for _ in range(36) for sh in QWEN3_4B_LAYER]
    plan = slime_amd.Fp8QuantPlan(ws, (128, 128))
    outs = plan.run()
    assert len(outs) == 252 and plan.total_tiles == 221760
    for i, (w, (q, s)) in enumerate(zip(ws, outs)):
        # reconstruction: half an e4m3 step of the block (the step at the top binade is 32 * scale)
        step = s.repeat_interleave(128, 0)[: w.shape[0]].repeat_interleave(128, 1)[:, : w.shape[1]] * 32
        assert ((q.float() * step / 32 - w.float()).abs() <= step / 2 * 1.001).all(), i
        if i % 9 == 0:          # 28 tensors: oracle on sampled 128-row stripes, bucket launch == single call
            for r0 in _stripe_rows(w.shape[0], cg):
                qo, so = C.fp8_block_quant(w[r0:r0 + 128].cpu(), (128, 128), plan.mode)
                assert torch.equal(q[r0:r0 + 128].cpu().view(torch.uint8), qo), (i, r0)
                assert torch.equal(s[r0 // 128].cpu().view(torch.int32), so[0].view(torch.int32)), (i, r0)
            q1, s1 = slime_amd.block_fp8(w, (128, 128))
            assert torch.equal(q1.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s1, s)
    # decode -> encode on the largest tensor: the dequantised bf16 weights give back the codes under the same scales
    # (bf16 rounding moves a value by 2^-9 of itself, far inside an e4m3 rounding interval)
    w, (q, s) = ws[4], outs[4]
    torch.set_default_dtype(torch.bfloat16)
    try:
        d = slime_amd.weight_dequant(q, s)
    finally:
        torch.set_default_dtype(torch.float32)
    back = (d.float() / s.repeat_interleave(128, 0).repeat_interleave(128, 1)).to(E4M3)
    assert torch.equal(back.view(torch.uint8) & 0x7F, q.view(torch.uint8) & 0x7F)      # sign of zero aside


def test_qwen3_30b_a3b_experts_int4(cuda):
    g = torch.Generator(device=cuda).manual_seed(1)
    cg = torch.Generator().manual_seed(1)
    layers, experts = 48, 128
    ws = []
    for _ in range(layers):
        gate, up = _gen((experts, 768, 2048), cuda, g, True), _gen((experts, 768, 2048), cuda, g, True)
        down = _gen((experts, 2048, 768), cuda, g, True)
        for e in range(experts):
            ws += [gate[e], up[e], down[e]]
    plan = slime_amd.Int4PackPlan(ws, 128)
    outs = plan.run()
    assert len(outs) == 18432
    picks = torch.randint(0, len(ws), (24,), generator=cg).tolist() + [0, len(ws) - 1]
    for i in picks:
        w, (p, s) = ws[i], outs[i]
        po, so, _ = C.int4_pack_layer(w.cpu().contiguous(), 128, True)
        assert torch.equal(p.cpu(), po) and torch.equal(s.cpu().view(torch.int16), so.view(torch.int16)), i
        p1, s1, _ = slime_amd.pack_layer(w, 128, True)
        assert torch.equal(p1, p) and torch.equal(s1.view(torch.int16), s.view(torch.int16))
    # reconstruction bound over every tensor of eight layers, through the INT4 -> bf16 kernel
    for i in range(0, 8 * 384):
        w, (p, s) = ws[i], outs[i]
        d = slime_amd.dequantize_int4(p, s, tuple(w.shape), 128)
        sf = s.float().repeat_interleave(128, dim=1)
        assert ((d.float() - w.float()).abs() <= sf * (0.5 + 7 * 2 ** -8) + d.float().abs() * 2.0 ** -8).all(), i


def test_deepseek_v3_layer_dequant(cuda):
    g = torch.Generator(device=cuda).manual_seed(2)
    cg = torch.Generator().manual_seed(2)
    xs, ss = [], []
    for shape in ((2048, 7168), (2048, 7168), (7168, 2048)):
        codes = torch.randint(0, 254, (256,) + shape, device=cuda, dtype=torch.uint8, generator=g)
        codes += (codes >= 0x7F).to(torch.uint8)
        sc = torch.exp(torch.empty((256, shape[0] // 128, shape[1] // 128), device=cuda).uniform_(-9.21034, -2.302585, generator=g))
        for e in range(256):
            xs.append(codes[e].view(E4M3))
            ss.append(sc[e])
    outs = slime_amd.Fp8DequantPlan(xs, ss).run()
    assert len(outs) == 768
    for i in torch.randint(0, 768, (12,), generator=cg).tolist() + [0, 767]:
        x, s, y = xs[i], ss[i], outs[i]
        r0 = int(torch.randint(0, x.shape[0] // 128, (1,), generator=cg)) * 128
        want = C.fp8_block_dequant(x[r0:r0 + 128].cpu().view(torch.uint8), s[r0 // 128:r0 // 128 + 1].cpu(), 128, 0)
        assert torch.equal(y[r0:r0 + 128].cpu().view(torch.int16), want.view(torch.int16)), i
        torch.set_default_dtype(torch.bfloat16)
        try:
            y1 = slime_amd.weight_dequant(x, s)
        finally:
            torch.set_default_dtype(torch.float32)
        assert torch.equal(y1.view(torch.int16), y.view(torch.int16))
    # decode -> encode: every finite code comes back when the bf16 value is quantised with the same scale
    x, s, y = xs[5], ss[5], outs[5]
    back = (y.float() / s.repeat_interleave(128, 0).repeat_interleave(128, 1)).to(E4M3)
    assert torch.equal(back.view(torch.uint8) & 0x7F, x.view(torch.uint8) & 0x7F)


@pytest.mark.parametrize("mode", [0, 2])
def test_qwen3_30b_a3b_state_dict_block_fp8(cuda, mode):
    """The FP8 launch of the benchmark's headline step at its full size: all 18 624 linear weights of the
    Qwen3-30B-A3B-shaped state dict (59.8 GB of bf16) through ONE launch, in the arithmetic the reference's own test
    runs (mode 0) and the one its tool runs on GPU tensors (mode 2)."""
    g = torch.Generator(device=cuda).manual_seed(3)
    cg = torch.Generator().manual_seed(3 + mode)
    layers, experts = 48, 128
    ws, attention = [], []
    for _ in range(layers):
        gate, up = _gen((experts, 768, 2048), cuda, g, True), _gen((experts, 768, 2048), cuda, g, True)
        down = _gen((experts, 2048, 768), cuda, g, True)
        for e in range(experts):
            ws += [gate[e], up[e], down[e]]
        for sh in ((4096, 2048), (512, 2048), (512, 2048), (2048, 4096)):
            attention.append(len(ws))
            ws.append(_gen(sh, cuda, g, False))
    plan = slime_amd.Fp8QuantPlan(ws, (128, 128), mode=mode)
    outs = plan.run()
    assert len(outs) == 18624 and plan.total_tiles == 1824768 and plan.bf16_bytes == 59793997824
    # oracle on whole expert tensors and on stripes of attention weights; the bucket launch equals the single call
    picks = torch.randint(0, len(ws), (20,), generator=cg).tolist() + [0, 1, 2, len(ws) - 5]
    picks += [attention[i] for i in torch.randint(0, len(attention), (8,), generator=cg).tolist()] + [len(ws) - 1]
    with slime_amd.torch_arithmetic("cpu" if mode == 0 else "device"):
        for i in picks:
            w, (q, s) = ws[i], outs[i]
            for r0 in _stripe_rows(w.shape[0], cg, n=2):
                qo, so = C.fp8_block_quant(w[r0:r0 + 128].cpu().contiguous(), (128, 128), mode)
                assert torch.equal(q[r0:r0 + 128].cpu().view(torch.uint8), qo), (i, r0)
                assert torch.equal(s[r0 // 128].cpu().view(torch.int32), so[0].view(torch.int32)), (i, r0)
            q1, s1 = slime_amd.block_fp8(w, (128, 128))
            assert torch.equal(q1.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s1, s), i
    # reconstruction bound over every tensor of three layers (first, middle, last)
    per_layer = 3 * experts + 4
    for layer in (0, layers // 2, layers - 1):
        for i in range(layer * per_layer, (layer + 1) * per_layer):
            w, (q, s) = ws[i], outs[i]
            step = s.repeat_interleave(128, 0)[: w.shape[0]].repeat_interleave(128, 1)[:, : w.shape[1]] * 32
            assert ((q.float() * step / 32 - w.float()).abs() <= step / 2 * 1.001).all(), i
    # nothing outside the sampled tensors was left unwritten: every scale of the bucket is a positive finite number
    scales = torch.cat([s.reshape(-1) for _, s in outs])
    assert scales.numel() == plan.total_tiles and bool(((scales > 0) & torch.isfinite(scales)).all())
