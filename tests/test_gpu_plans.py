"""The one-launch forms for many tensors against the per-tensor functions and the CPU oracle: asymmetric INT4 plan,
QAT forward over many weights, FP8 dequant with per-item descriptors, xor delta with per-chunk descriptors."""

import numpy as np
import pytest
import torch

import slime_amd
from oracle import c_oracle as C
from oracle import delta_ref as D
from slime_amd import delta
from slime_amd.int4 import fake_int4_quantization_ste_many
from tests import wq_inputs as I

pytestmark = pytest.mark.gpu
E4M3 = torch.float8_e4m3fn


@pytest.mark.parametrize("gs", [128, 32])
def test_asym_pack_plan_equals_pack_layer_and_oracle(cuda, gs):
    shapes = [(96, 256), (40, 768), (8, 128), (64, 128), (16, 7168), (128, 2048), (200, 1024)] * 3
    ws = [I.weights(*sh, seed=400 + i, outlier_p=0.01) for i, sh in enumerate(shapes)]
    ws[3] = ws[3].abs() + 0.5                      # a one-sided tensor: codes above 15, packed unmasked
    plan = slime_amd.Int4PackPlan([w.to(cuda) for w in ws], gs, sym=False)
    for _ in range(2):
        outs = plan.run()
        for w, (p, s, z) in zip(ws, outs):
            po, so, zo = C.int4_pack_layer(w, gs, False)
            assert torch.equal(p.cpu(), po) and I.same_bits(s.cpu(), so) and torch.equal(z.cpu(), zo)
    p1, s1, z1 = slime_amd.pack_layer(ws[0].to(cuda), gs, False)
    assert torch.equal(p1, outs[0][0]) and torch.equal(z1, outs[0][2])
    with pytest.raises(ValueError, match="multiple of 8"):
        slime_amd.Int4PackPlan([I.weights(12, 256, seed=1).to(cuda)], gs, sym=False)


def test_ste_many_equals_single_calls(cuda):
    shapes = [(96, 256), (33, 768), (1, 128), (7, 7168), (128, 2048), (63, 128)] * 4
    ws = [I.weights(*sh, seed=500 + i) for i, sh in enumerate(shapes)]
    wg = [w.to(cuda).requires_grad_() for w in ws]
    wg[2].main_grad = torch.zeros(1, device=cuda)
    for arith, div7 in (("device", 1), ("cpu", 0)):
        with slime_amd.torch_arithmetic(arith):
            outs = fake_int4_quantization_ste_many(wg, 128)
            for w, g, o in zip(ws, wg, outs):
                assert I.same_bits(o.detach().cpu(), C.int4_fake_ste(w, 128, div7))
                assert I.same_bits(o.detach().cpu(), slime_amd.fake_int4_quantization_ste(g, 128).detach().cpu())
    assert outs[2].main_grad is wg[2].main_grad
    sum((o.float() * (i + 1)).sum() for i, o in enumerate(outs)).backward()     # straight-through: d out / d w = 1
    for i, g in enumerate(wg):
        assert torch.equal(g.grad, torch.full_like(g, float(i + 1)))
    # weights outside the fast layout fall back to one call each
    odd = [I.weights(8, 100, seed=1).to(cuda), wg[0].detach()]
    outs = fake_int4_quantization_ste_many(odd, 32)
    assert I.same_bits(outs[0].cpu(), slime_amd.fake_int4_quantization_ste(odd[0], 32).cpu())
    assert fake_int4_quantization_ste_many([], 128) == []
    plan = slime_amd.Int4StePlan([w.to(cuda) for w in ws], 128)
    for w, o in zip(ws, plan.run()):
        assert I.same_bits(o.cpu(), C.int4_fake_ste(w, 128, 1))
    with pytest.raises(ValueError):
        slime_amd.Int4StePlan(odd, 32)


def test_dequant_plan_many_tensors_uses_item_table(cuda):
    shapes = [(256, 384), (300, 200), (7, 7168), (129, 1), (128, 128), (16, 1024), (17, 1040), (5, 1000), (640, 512)] * 8
    xs = [I.fp8_codes(*sh, seed=i) for i, sh in enumerate(shapes)]
    ss = [I.log_uniform_scales(-(-sh[0] // 128), -(-sh[1] // 128), seed=i) for i, sh in enumerate(shapes)]
    for mode in (0, 1):
        plan = slime_amd.Fp8DequantPlan([x.to(cuda).view(E4M3) for x in xs], [s.to(cuda) for s in ss], 128, mode)
        assert plan._items is not None and plan._items.shape == (plan.total_work, 6)
        for x, s, y in zip(xs, ss, plan.run()):
            assert I.same_bits(y.cpu(), C.fp8_block_dequant(x, s, 128, mode))
    plan = slime_amd.Fp8DequantPlan([x.to(cuda).view(E4M3) for x in xs], [s.to(cuda) for s in ss], 128, 0, torch.float32)
    y = plan.run()[1]
    assert y.dtype == torch.float32 and torch.equal(y.cpu(), xs[1].view(E4M3).float() * ss[1].repeat_interleave(128, 0)[:300].repeat_interleave(128, 1)[:, :200])


def test_xor_diff_plan_equals_many_and_reference(cuda):
    rng = np.random.default_rng(5)
    sizes = [0, 1, 15, 16, 17, 4096, 16384, 16385, 65521, 100000, (1 << 20) + 3, 16384 * 40 + 7] * 6
    olds_np = [rng.integers(0, 256, n, dtype=np.uint8) for n in sizes]
    news_np = []
    for i, o in enumerate(olds_np):
        nw = o.copy()
        if i % 3 and o.size:
            idx = rng.random(o.size) < 0.05
            nw[idx] ^= rng.integers(1, 256, int(idx.sum()), dtype=np.uint8)
        news_np.append(nw)
    news = [torch.from_numpy(x).to(cuda) for x in news_np]
    olds = [torch.from_numpy(x).to(cuda) for x in olds_np]
    plan = delta.XorDiffPlan(news, olds)
    diffs, results = plan.run(update_snapshot=False)
    d2, r2 = delta.xor_diff_many(news, olds)
    assert torch.equal(results, r2.to(results.device))
    for i, (nw, od) in enumerate(zip(news_np, olds_np)):
        want, changed = D.xor_delta_ref(nw, od)
        assert np.array_equal(diffs[i].cpu().numpy(), want) and torch.equal(diffs[i], d2[i]), i
        assert results[i].tolist() == [changed, int(D.adler32_ref(nw), 16)], i
        assert np.array_equal(olds[i].cpu().numpy(), od)
    plan.run(update_snapshot=True)                      # second run of the same table, now bringing the snapshots up to date
    for nw, od in zip(news_np, olds):
        assert np.array_equal(od.cpu().numpy(), nw)
    _, results = plan.run()
    assert results[:, 0].sum().item() == 0              # nothing differs any more
    counts_only = delta.XorDiffPlan(news, olds, want_diff=False)
    assert counts_only.run()[0] is None and counts_only.results[:, 1].tolist() == results[:, 1].tolist()
