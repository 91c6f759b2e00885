"""Name routing of the quantise-on-update step (CPU; the quantisers themselves are stubbed)."""

import pytest
import torch

import slime_amd.processors as P

FP8_CFG = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic", "weight_block_size": [128, 128]}
L = "module.module.decoder.layers.3."


@pytest.fixture
def stub(monkeypatch):
    calls = []

    def fake_block(w, bs):
        calls.append(("block", tuple(bs)))
        return w.to(torch.float32), torch.ones(1, 1)

    def fake_tensor(w):
        calls.append(("tensor",))
        return w.to(torch.float32), torch.ones(1)

    monkeypatch.setattr(P, "blockwise_cast_to_fp8_triton", fake_block)
    monkeypatch.setattr(P, "tensor_fp8", fake_tensor)
    return calls


def _w():
    return torch.zeros(4, 4, dtype=torch.bfloat16)


QUANTIZED = [
    L + "self_attention.linear_qkv.weight", L + "self_attention.linear_proj.weight",
    L + "mlp.linear_fc1.weight", L + "mlp.linear_fc2.weight",
    L + "mlp.experts.linear_fc1.weight17", L + "mlp.experts.linear_fc2.weight0",
    L + "mlp.shared_experts.linear_fc1.weight", L + "mlp.shared_experts.linear_fc2.weight",
    L + "self_attention.linear_q_down_proj.weight", L + "self_attention.linear_kv_up_proj.weight",
    L + "self_attention.wq_b.weight", L + "self_attention.linear_attn.out_proj.weight",
    "module.module.mtp.layers.0.transformer_layer.mlp.linear_fc1.weight",
]
PASSED_THROUGH = [
    "module.module.embedding.word_embeddings.weight", "module.module.output_layer.weight",
    "module.module.decoder.final_layernorm.weight", L + "mlp.router.weight",
    L + "self_attention.linear_qkv.layer_norm_weight", L + "self_attention.q_layernorm.weight",
    L + "mlp.experts.router.weight3", L + "mlp.shared_experts.gate_weight",
    L + "self_attention.linear_qkv.bias", "module.module.mtp.layers.0.enorm.weight",
]


@pytest.mark.parametrize("name", QUANTIZED)
def test_fp8_quantized_names(stub, name):
    params = [("model.layers.3.x.weight", _w())]
    out = P.quantize_params(None, name, params, FP8_CFG)
    assert [n for n, _ in out] == ["model.layers.3.x.weight", "model.layers.3.x.weight_scale_inv"]
    assert stub == [("block", (128, 128))]


@pytest.mark.parametrize("name", PASSED_THROUGH)
def test_fp8_passthrough_names(stub, name):
    params = [("a.weight", _w())]
    assert P.quantize_params(None, name, params, FP8_CFG) is params
    assert stub == []


def test_fp8_expert_scales_are_dropped(stub):
    params = [("e.gate_proj.weight", _w()), ("e.gate_proj.weight_scale", _w()), ("e.up_proj.weight", _w())]
    out = P.quantize_params_fp8(None, L + "mlp.experts.linear_fc1.weight2", params, FP8_CFG)
    assert [n for n, _ in out] == ["e.gate_proj.weight", "e.gate_proj.weight_scale_inv",
                                   "e.up_proj.weight", "e.up_proj.weight_scale_inv"]


def test_fp8_per_tensor_branch(stub):
    cfg = dict(FP8_CFG, weight_block_size=None)
    out = P.quantize_params_fp8(None, L + "mlp.linear_fc2.weight", [("d.weight", _w())], cfg)
    assert [n for n, _ in out] == ["d.weight", "d.weight_scale"] and stub == [("tensor",)]


def test_fp8_config_asserts():
    with pytest.raises(AssertionError):
        P.quantize_params_fp8(None, "x", [], dict(FP8_CFG, fmt="e5m2"))
    with pytest.raises(AssertionError):
        P.quantize_params_fp8(None, "x", [], dict(FP8_CFG, activation_scheme="static"))
    with pytest.raises(AssertionError):
        P._quantize_param("model.bias", _w(), [128, 128])


def test_dispatch_none_and_unknown():
    params = [("a.weight", _w())]
    assert P.quantize_params(None, "x", params, None) is params
    assert P.quantize_params(None, "x", params, {"quant_method": "mxfp4"}) is params


def test_compressed_tensors_routing(monkeypatch):
    seen = []

    def fake_pack(w, gs, sym):
        seen.append((tuple(w.shape), gs, sym))
        return torch.zeros(1, dtype=torch.int32), torch.zeros(1), (None if sym else torch.zeros(1, dtype=torch.int32))

    monkeypatch.setattr(P, "pack_layer", fake_pack)
    cfg = {"quant_method": "compressed-tensors",
           "config_groups": {"group_0": {"weights": {"group_size": 128, "symmetric": True}}},
           "ignore": ["lm_head", "re:.*self_attn.*", "model.layers.0.mlp.experts.3.down_proj.weight"]}
    params = [("model.layers.0.mlp.experts.0.gate_proj.weight", torch.zeros(8, 128)),
              ("model.layers.0.self_attn.q_proj.weight", torch.zeros(8, 128)),
              ("lm_head.weight", torch.zeros(8, 128)),
              ("model.layers.0.mlp.experts.3.down_proj.weight", torch.zeros(8, 128)),
              ("model.layers.0.mlp.experts.0.gate_proj.bias", torch.zeros(8, 128)),
              ("model.layers.0.input_layernorm.weight", torch.zeros(128))]
    out = P.quantize_params(None, "whatever", params, cfg)
    names = [n for n, _ in out]
    assert names == ["model.layers.0.mlp.experts.0.gate_proj.weight_packed",
                     "model.layers.0.mlp.experts.0.gate_proj.weight_scale",
                     "model.layers.0.mlp.experts.0.gate_proj.weight_shape",
                     "model.layers.0.self_attn.q_proj.weight", "lm_head.weight",
                     "model.layers.0.mlp.experts.3.down_proj.weight",
                     "model.layers.0.mlp.experts.0.gate_proj.bias", "model.layers.0.input_layernorm.weight"]
    assert seen == [((8, 128), 128, True)]
    shape = dict(out)["model.layers.0.mlp.experts.0.gate_proj.weight_shape"]
    assert shape.dtype == torch.int32 and shape.tolist() == [8, 128]
    # asymmetric: zero point comes first
    cfg["config_groups"]["group_0"]["weights"]["symmetric"] = False
    out = P.quantize_params(None, "whatever", params[:1], cfg)
    assert [n.rsplit(".", 1)[1] for n, _ in out] == ["weight_zero_point", "weight_packed", "weight_scale", "weight_shape"]
