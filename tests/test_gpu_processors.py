"""quantize_params on the GPU: state-dict layout and bytes for the FP8 and INT4 weight-sync branches."""

import pytest
import torch

import slime_amd
from oracle import c_oracle as C
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
