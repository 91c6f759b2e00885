"""quantize_params on the GPU: state-dict layout and bytes for the FP8 and INT4 weight-sync branches."""

import pytest
import torch

import slime_amd
from oracle import c_oracle as C
from slime_amd import processors
from tests import wq_inputs as I

pytestmark = pytest.mark.gpu
L = "module.module.decoder.layers.0."


def test_fp8_qkv_params(cuda):
    cfg = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic", "weight_block_size": [128, 128]}
    ws = {"q_proj": I.weights(4096, 2560, seed=1), "k_proj": I.weights(1024, 2560, seed=2),
          "v_proj": I.weights(1024, 2560, seed=3)}
    params = [(f"model.layers.0.self_attn.{n}.weight", w.to(cuda)) for n, w in ws.items()]
    out = slime_amd.quantize_params(None, L + "self_attention.linear_qkv.weight", params, cfg)
    assert [n for n, _ in out] == [f"model.layers.0.self_attn.{n}.{suffix}" for n in ws
                                   for suffix in ("weight", "weight_scale_inv")]
    d = dict(out)
    for n, w in ws.items():
        qo, so = C.fp8_block_quant(w, (128, 128), 1)       # the weight-sync path uses the reciprocal-multiply variant
        q, s = d[f"model.layers.0.self_attn.{n}.weight"], d[f"model.layers.0.self_attn.{n}.weight_scale_inv"]
        assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.float32
        assert torch.equal(q.cpu().view(torch.uint8), qo) and I.same_bits(s.cpu(), so)
    # single tensor, per-tensor scale
    cfg2 = dict(cfg, weight_block_size=None)
    out = slime_amd.quantize_params(None, L + "mlp.linear_fc2.weight", [("model.layers.0.mlp.down_proj.weight",
                                                                         ws["k_proj"].to(cuda))], cfg2)
    assert [n for n, _ in out] == ["model.layers.0.mlp.down_proj.weight", "model.layers.0.mlp.down_proj.weight_scale"]
    qo, so = C.fp8_tensor_quant(ws["k_proj"], 2)
    assert torch.equal(out[0][1].cpu().view(torch.uint8), qo) and I.same_bits(out[1][1].cpu(), so)
    # untouched parameter: same list object comes back
    p = [("model.embed_tokens.weight", ws["k_proj"].to(cuda))]
    assert slime_amd.quantize_params(None, "module.module.embedding.word_embeddings.weight", p, cfg) is p


def test_int4_expert_params(cuda):
    cfg = {"quant_method": "compressed-tensors",
           "config_groups": {"group_0": {"weights": {"group_size": 128, "symmetric": True}}},
           "ignore": ["lm_head", "re:.*self_attn.*", "re:.*shared_experts.*"]}
    w = I.weights(768, 2048, seed=5)
    params = [("model.layers.0.mlp.experts.7.gate_proj.weight", w.to(cuda)),
              ("model.layers.0.self_attn.o_proj.weight", w.to(cuda))]
    out = slime_amd.quantize_params(None, L + "mlp.experts.linear_fc1.weight7", params, cfg)
    names = [n for n, _ in out]
    base = "model.layers.0.mlp.experts.7.gate_proj."
    assert names == [base + "weight_packed", base + "weight_scale", base + "weight_shape",
                     "model.layers.0.self_attn.o_proj.weight"]
    d = dict(out)
    po, so, _ = C.int4_pack_layer(w, 128, True)
    assert torch.equal(d[base + "weight_packed"].cpu(), po) and I.same_bits(d[base + "weight_scale"].cpu(), so)
    assert d[base + "weight_shape"].tolist() == [768, 2048] and d[base + "weight_shape"].dtype == torch.int32
    assert d[base + "weight_shape"].is_cuda


def test_shim_module_and_hook(cuda):
    import slime_amd.fake_int4_quant_cuda as shim

    w = I.weights(8, 256, seed=1)
    q, s, z = shim.fake_int4_quant_cuda(w.to(cuda), (1, 128), True)
    qo, so, zo = C.int4_fake_quant(w, (1, 128), True)
    assert I.same_bits(q.cpu(), qo) and I.same_bits(s.cpu(), so)
    qw, sc = slime_amd.quantize_weight(w.to(cuda), (128, 128))
    assert tuple(qw.shape) == (8, 256) and tuple(sc.shape) == (1, 2) and sc.dtype == torch.float32


@pytest.mark.parametrize("shape", [(768, 2048), (300, 200), (129, 127)])
@pytest.mark.parametrize("ue8m0", [False, True])
def test_quantize_grouped_weights_equals_the_per_expert_loop(cuda, shape, ue8m0):
    """The stacked [E, N, K] codes and [E, n, k] scales of the alignment forward's grouped weights, one launch, against
    the loop it replaces (quantise each expert, copy into the stack) and the oracle."""
    E = 5
    fc = I.weights(E * shape[0], shape[1], seed=shape[0]).to(cuda)
    views = list(fc.chunk(E, dim=0))                                  # expert weights as views of one parameter
    views[2] = views[2].clone().t().contiguous().t()                  # one of them column-major
    q, s = slime_amd.quantize_grouped_weights(views, (128, 128), use_ue8m0=ue8m0)
    tm, tn = -(-shape[0] // 128), -(-shape[1] // 128)
    assert q.shape == (E, *shape) and q.dtype == torch.float8_e4m3fn and s.shape == (E, tm, tn) and s.dtype == torch.float32
    assert q.is_contiguous() and s.is_contiguous()
    one = slime_amd.quant_weight_ue8m0 if ue8m0 else slime_amd.blockwise_cast_to_fp8_triton
    for e, w in enumerate(views):
        qe, se = one(w.contiguous(), [128, 128])
        assert I.same_bits(q[e].view(torch.uint8), qe.view(torch.uint8)) and I.same_bits(s[e], se), e
        qo, so = C.fp8_block_quant(w.cpu().contiguous(), (128, 128), 3 if ue8m0 else 1)
        assert torch.equal(q[e].cpu().view(torch.uint8), qo) and I.same_bits(s[e].cpu(), so), e
    info = processors.plan_cache_info()
    q2, _ = slime_amd.quantize_grouped_weights(views, (128, 128), use_ue8m0=ue8m0)
    after = processors.plan_cache_info()
    assert (after["builds"], after["resolves"]) == (info["builds"], info["resolves"])      # same weights: nothing to do
    assert I.same_bits(q2.view(torch.uint8), q.view(torch.uint8))
    assert q2.data_ptr() != q.data_ptr()                              # fresh outputs on every call
    # the same grouped linear somewhere else (freshly gathered weights): the layout is reused, the addresses resolved again
    moved = [w.clone(memory_format=torch.preserve_format) for w in views]
    assert [w.stride() for w in moved] == [w.stride() for w in views] and moved[0].data_ptr() != views[0].data_ptr()
    q3, s3 = slime_amd.quantize_grouped_weights(moved, (128, 128), use_ue8m0=ue8m0)
    last = processors.plan_cache_info()
    assert last["builds"] == info["builds"] and last["resolves"] == info["resolves"] + 1
    assert I.same_bits(q3.view(torch.uint8), q.view(torch.uint8)) and I.same_bits(s3, s)


def test_quantize_grouped_weights_argument_errors(cuda):
    w = I.weights(128, 256).to(cuda)
    with pytest.raises(RuntimeError, match="must be BF16"):
        slime_amd.quantize_grouped_weights([w, w.float()])
    with pytest.raises(RuntimeError, match="expected"):
        slime_amd.quantize_grouped_weights([w, w[:64]])
    with pytest.raises(RuntimeError, match="must be on"):
        slime_amd.quantize_grouped_weights([w, w.cpu()])
    with pytest.raises(ValueError):
        slime_amd.quantize_grouped_weights([])
    q, s = slime_amd.quantize_grouped_weights([w[:0], w[:0]])
    assert q.shape == (2, 0, 256) and s.shape == (2, 0, 2)


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_few_tensor_launch_through_the_c_abi(cuda, mode):
    """wq_fp8_block_quant_few: up to four descriptors in the kernel arguments - ragged and strided members, an empty one
    in the middle, absolute output addresses (out_base NULL) and offsets from a base, every arithmetic mode."""
    import ctypes

    from slime_amd import _lib
    from slime_amd.processors import _QuantDesc

    ws = [I.weights(300, 520, seed=61), I.weights(128, 128, seed=62), I.weights(0, 256, seed=63), I.weights(264, 512, seed=64)[:, ::2]]
    wg = [w.to(cuda) for w in ws[:3]] + [I.weights(264, 512, seed=64).to(cuda)[:, ::2]]
    lib = _lib.load()
    for with_base in (False, True):
        outs, descs, off = [], (_QuantDesc * 4)(), 0
        flat = torch.full((1 << 20,), 0xEE, dtype=torch.uint8, device=cuda)
        for d, w in zip(descs, wg):
            M, N = w.shape
            tm, tn = -(-M // 128), -(-N // 128)
            q0, s0 = off, (off + M * N + 127) // 128 * 128
            off = (s0 + 4 * tm * tn + 127) // 128 * 128
            base = 0 if with_base else flat.data_ptr()
            d.x, d.y, d.s, d.M, d.N, d.sx_m, d.sx_n, d.sy_m = w.data_ptr() if M else 0, base + q0, base + s0, M, N, w.stride(0), w.stride(1), N
            outs.append((q0, s0, M, N, tm, tn))
        rc = lib.wq_fp8_block_quant_few(descs, 4, flat.data_ptr() if with_base else None, 128, 128, mode, _lib.stream_ptr(cuda))
        _lib.check(rc, "few")
        host = flat.cpu()
        for w, (q0, s0, M, N, tm, tn) in zip(ws, outs):
            if M == 0:
                continue
            qo, so = C.fp8_block_quant(w.contiguous(), (128, 128), mode)
            assert torch.equal(host[q0:q0 + M * N].view(M, N), qo), (mode, with_base, M, N)
            assert torch.equal(host[s0:s0 + 4 * tm * tn].clone().view(torch.int32).view(tm, tn), so.view(torch.int32)), (mode, with_base, M, N)
        assert bool((host[off:] == 0xEE).all())
    assert lib.wq_fp8_block_quant_few(descs, 5, None, 128, 128, mode, None) == -2
