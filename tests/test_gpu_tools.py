"""Offline converters end to end on a tiny synthetic HF checkpoint: file formats and bytes."""

import json
import os

import pytest
import torch
from safetensors import safe_open
from safetensors.torch import load_file, save_file

from oracle import c_oracle as C
from slime_amd.tools import convert_hf_to_fp8 as F8
from slime_amd.tools import convert_hf_to_int4_direct as I4
from slime_amd.tools import convert_k2_thinking_int4_to_bf16 as K2
from slime_amd.tools import fp8_cast_bf16 as CAST
from tests import wq_inputs as I

pytestmark = pytest.mark.gpu


@pytest.fixture
def ckpt(tmp_path):
    d = tmp_path / "bf16"
    d.mkdir()
    s1 = {"model.embed_tokens.weight": I.weights(64, 256, seed=1),
          "model.layers.0.self_attn.q_proj.weight": I.weights(384, 256, seed=2),
          "model.layers.0.self_attn.q_norm.weight": torch.ones(128, dtype=torch.bfloat16),
          "model.layers.0.mlp.gate.weight": I.weights(8, 256, seed=3),
          # 296 rows: ragged for 128x128 blocks, and a multiple of 8 as asymmetric zero-point packing needs
          "model.layers.0.mlp.experts.0.gate_proj.weight": I.weights(296, 256, seed=4),
          "model.layers.0.mlp.experts.0.down_proj.weight": I.weights(256, 384, seed=5)}
    s2 = {"model.layers.1.mlp.experts.1.up_proj.weight": I.weights(128, 128, seed=6),
          "model.layers.1.self_attn.o_proj.bias": torch.zeros(256, dtype=torch.bfloat16),
          "lm_head.weight": I.weights(64, 256, seed=7)}
    save_file(s1, str(d / "model-00001-of-00002.safetensors"), metadata={"format": "pt"})
    save_file(s2, str(d / "model-00002-of-00002.safetensors"), metadata={"format": "pt"})
    json.dump({"architectures": ["Qwen3MoeForCausalLM"], "hidden_size": 256}, open(d / "config.json", "w"))
    (d / "tokenizer.json").write_text("{}")
    (d / "sub").mkdir()
    return d, {**s1, **s2}


def test_convert_hf_to_fp8_block_and_cast_back(ckpt, tmp_path, cuda):
    src, tensors = ckpt
    out = tmp_path / "fp8"
    F8.main(["--model-dir", str(src), "--save-dir", str(out), "--strategy", "block", "--block-size", "128", "128"])
    assert sorted(os.listdir(out)) == ["config.json", "model-00001-of-00002.safetensors",
                                       "model-00002-of-00002.safetensors", "model.safetensors.index.json",
                                       "tokenizer.json"]
    cfg = json.load(open(out / "config.json"))
    q = cfg["quantization_config"]
    assert q["quant_method"] == "fp8" and q["fmt"] == "e4m3" and q["activation_scheme"] == "dynamic"
    assert q["weight_block_size"] == [128, 128] and cfg["hidden_size"] == 256
    assert q["modules_to_not_convert"] == sorted({"model.embed_tokens", "model.layers.0.self_attn.q_norm",
                                                  "model.layers.0.mlp.gate", "model.layers.1.self_attn.o_proj.bias",
                                                  "lm_head"})
    idx = json.load(open(out / "model.safetensors.index.json"))
    got = {}
    for f in ("model-00001-of-00002.safetensors", "model-00002-of-00002.safetensors"):
        with safe_open(str(out / f), framework="pt") as h:
            assert h.metadata() == {"format": "pt"}
        for k, v in load_file(str(out / f)).items():
            got[k] = v
            assert idx["weight_map"][k] == f
    assert set(idx["weight_map"]) == set(got)
    assert idx["metadata"]["total_size"] == sum(len(v) for v in got.values())
    converted = [k for k in tensors if F8.is_converted(k)]
    assert len(converted) == 4
    for k, w in tensors.items():
        if k in converted:
            qo, so = C.fp8_block_quant(w, (128, 128), 2)
            assert got[k].dtype == torch.float8_e4m3fn and torch.equal(got[k].view(torch.uint8), qo), k
            s = got[k.replace(".weight", ".weight_scale_inv")]
            assert s.dtype == torch.float32 and torch.equal(s.view(torch.int32), so.view(torch.int32)), k
        else:
            assert I.same_bits(got[k], w), k
    # key order inside a shard: converted weight directly followed by its scale
    with safe_open(str(out / "model-00001-of-00002.safetensors"), framework="pt") as h:
        assert "model.layers.0.self_attn.q_proj.weight_scale_inv" in h.keys()

    back = tmp_path / "bf16_again"
    CAST.main(str(out), str(back))
    assert sorted(os.listdir(back)) == ["config.json", "model-00001-of-00002.safetensors",
                                        "model-00002-of-00002.safetensors", "model.safetensors.index.json",
                                        "tokenizer.json"]
    idx2 = json.load(open(back / "model.safetensors.index.json"))
    assert idx2["metadata"] == {} and not any(k.endswith("_scale_inv") for k in idx2["weight_map"])
    assert set(idx2["weight_map"]) == set(tensors)
    for f in ("model-00001-of-00002.safetensors", "model-00002-of-00002.safetensors"):
        for k, v in load_file(str(back / f)).items():
            if k in converted:
                want = C.fp8_block_dequant(got[k].view(torch.uint8), got[k.replace(".weight", ".weight_scale_inv")], 128, 0)
                assert v.dtype == torch.bfloat16 and I.same_bits(v, want), k
            else:
                assert I.same_bits(v, tensors[k]), k


@pytest.mark.parametrize("strategy", ["tensor", "channel"])
def test_convert_hf_to_fp8_other_strategies(ckpt, tmp_path, cuda, strategy):
    src, tensors = ckpt
    out = tmp_path / strategy
    F8.main(["--model-dir", str(src), "--save-dir", str(out), "--strategy", strategy])
    got = {}
    for f in ("model-00001-of-00002.safetensors", "model-00002-of-00002.safetensors"):
        got.update(load_file(str(out / f)))
    k = "model.layers.0.mlp.experts.0.gate_proj.weight"
    qo, so = (C.fp8_tensor_quant if strategy == "tensor" else C.fp8_channel_quant)(tensors[k], 2)
    assert torch.equal(got[k].view(torch.uint8), qo)
    s = got[k.replace(".weight", ".weight_scale")]
    assert s.shape == so.shape and torch.equal(s.view(torch.int32), so.view(torch.int32))
    q = json.load(open(out / "config.json"))["quantization_config"]
    assert (q["quant_method"] == "fp8") == (strategy == "tensor")


@pytest.mark.parametrize("strategy", ["block", "tensor", "channel"])
def test_convert_hf_to_fp8_half_and_single_precision_checkpoints(tmp_path, cuda, strategy):
    """The reference's quant_fp8 takes whatever float dtype the checkpoint holds; so does the converter."""
    src, out = tmp_path / "mixed", tmp_path / f"mixed_{strategy}"
    src.mkdir()
    tensors = {"model.layers.0.self_attn.q_proj.weight": I.weights(300, 256, seed=2).to(torch.float16),
               "model.layers.0.self_attn.o_proj.weight": I.weights(256, 384, seed=3).float() * 1.001,
               "model.layers.0.mlp.down_proj.weight": I.weights(128, 256, seed=4)}
    save_file(tensors, str(src / "model.safetensors"), metadata={"format": "pt"})
    json.dump({"architectures": ["X"]}, open(src / "config.json", "w"))
    F8.main(["--model-dir", str(src), "--save-dir", str(out), "--strategy", strategy] +
            (["--block-size", "128", "128"] if strategy == "block" else []))
    got = load_file(str(out / "model.safetensors"))
    for k, w in tensors.items():
        qo, so = {"block": lambda t: C.fp8_block_quant(t, (128, 128), 2), "tensor": lambda t: C.fp8_tensor_quant(t, 2),
                  "channel": lambda t: C.fp8_channel_quant(t, 2)}[strategy](w)
        s = got[k.replace(".weight", ".weight_scale_inv" if strategy == "block" else ".weight_scale")]
        assert got[k].dtype == torch.float8_e4m3fn and torch.equal(got[k].view(torch.uint8), qo), k
        assert s.shape == so.shape and torch.equal(s.view(torch.int32), so.view(torch.int32)), k


@pytest.mark.parametrize("group,sym", [(128, True), (32, True), (128, False)])
def test_convert_hf_to_int4_direct(ckpt, tmp_path, cuda, group, sym):
    src, tensors = ckpt
    out = tmp_path / f"int4_{group}_{sym}"
    argv = ["--model-dir", str(src), "--save-dir", str(out), "--group-size", str(group)] + (["--is-symmetric"] if sym else [])
    I4.main(argv)
    cfg = json.load(open(out / "config.json"))["quantization_config"]
    assert cfg["format"] == "pack-quantized" and cfg["config_groups"]["group_0"]["weights"]["group_size"] == group
    assert cfg["config_groups"]["group_0"]["weights"]["symmetric"] is sym and cfg["ignore"] == I4.DEFAULT_IGNORE_RULES
    got = {}
    for f in ("model-00001-of-00002.safetensors", "model-00002-of-00002.safetensors"):
        got.update(load_file(str(out / f)))
    packed_names = [k for k in tensors if not I4.is_ignored(k, I4.DEFAULT_IGNORE_RULES) and k.endswith(".weight")
                    and tensors[k].dim() >= 2]
    assert sorted(packed_names) == ["model.layers.0.mlp.experts.0.down_proj.weight",
                                    "model.layers.0.mlp.experts.0.gate_proj.weight",
                                    "model.layers.1.mlp.experts.1.up_proj.weight"]
    for k, w in tensors.items():
        if k in packed_names:
            po, so, zo = C.int4_pack_layer(w, group, sym)
            assert k not in got
            assert torch.equal(got[k.replace(".weight", ".weight_packed")], po), k
            assert I.same_bits(got[k.replace(".weight", ".weight_scale")], so), k
            assert got[k.replace(".weight", ".weight_shape")].tolist() == list(w.shape)
            assert got[k.replace(".weight", ".weight_shape")].dtype == torch.int32
            if sym:
                assert k.replace(".weight", ".weight_zero_point") not in got
            else:
                assert torch.equal(got[k.replace(".weight", ".weight_zero_point")], zo), k
        else:
            assert I.same_bits(got[k], w), k
    idx = json.load(open(out / "model.safetensors.index.json"))
    assert set(idx["weight_map"]) == set(got) and idx["metadata"]["total_size"] == sum(len(v) for v in got.values())


def test_convert_int4_experts_to_bf16(tmp_path, cuda):
    # a pack-quantized checkpoint as convert_hf_to_int4_direct writes it -> bf16, tool against the oracle
    src = tmp_path / "int4"
    src.mkdir()
    w = {"model.layers.0.mlp.experts.0.gate_proj": I.weights(64, 256, seed=1),
         "model.layers.0.mlp.experts.0.down_proj": I.weights(256, 128, seed=2),
         "model.layers.0.mlp.experts.1.up_proj": I.weights(40, 384, seed=3)}
    shard = {"model.embed_tokens.weight": I.weights(16, 64, seed=4),
             "model.layers.0.mlp.shared_experts.gate_proj.weight_packed": torch.zeros(4, 8, dtype=torch.int32),
             "model.layers.0.mlp.experts.2.up_proj.weight_packed": torch.ones(4, 8, dtype=torch.int32)}   # incomplete
    want = {}
    for name, t in w.items():
        p, s, _ = C.int4_pack_layer(t, 64, True)
        shard[f"{name}.weight_packed"], shard[f"{name}.weight_scale"] = p, s
        shard[f"{name}.weight_shape"] = torch.tensor(list(t.shape), dtype=torch.int32)
        want[f"{name}.weight"] = C.int4_dequant(p, s, tuple(t.shape), 64)
    save_file(shard, str(src / "model-00001-of-00001.safetensors"))
    cfg = {"hidden_size": 256, "moe_intermediate_size": 64,
           "quantization_config": {"config_groups": {"group_0": {"weights": {"group_size": 64}}}}}
    json.dump(cfg, open(src / "config.json", "w"))
    (src / "tokenizer.json").write_text("{}")
    (src / "modeling.py").write_text("# code")
    (src / "notes.txt").write_text("not copied")
    out = tmp_path / "bf16"
    assert K2._load_config(str(src), None) == (256, 64, 64)
    K2.main(["--model-dir", str(src), "--output-dir", str(out)])
    got = load_file(str(out / "model-00001-of-00001.safetensors"))
    for name, t in want.items():
        assert got[name].dtype == torch.bfloat16 and I.same_bits(got[name], t), name
    assert not any(k.endswith((".weight_scale", ".weight_shape")) for k in got)
    assert torch.equal(got["model.embed_tokens.weight"], shard["model.embed_tokens.weight"])
    assert "model.layers.0.mlp.shared_experts.gate_proj.weight_packed" in got            # shared experts are not touched
    assert "model.layers.0.mlp.experts.2.up_proj.weight_packed" in got                   # incomplete triple is kept
    index = json.load(open(out / "model.safetensors.index.json"))
    assert index["metadata"] == {} and set(index["weight_map"]) == set(got)
    assert sorted(os.listdir(out)) == ["config.json", "model-00001-of-00001.safetensors", "model.safetensors.index.json",
                                       "modeling.py", "tokenizer.json"]
    # skip_existing: a second run leaves the file alone; --overwrite rewrites it
    before = os.path.getmtime(out / "model-00001-of-00001.safetensors")
    K2.main(["--model-dir", str(src), "--output-dir", str(out)])
    assert os.path.getmtime(out / "model-00001-of-00001.safetensors") == before


def test_convert_int4_experts_with_other_scale_dtypes(tmp_path, cuda):
    # the reference converts whatever scale dtype the shard holds with .to(float32) (:150): fp16 and fp32 scales go
    # through, each against the oracle with that dtype's arithmetic; bf16 members of the same shard share one launch
    src = tmp_path / "int4"
    src.mkdir()
    shard, want = {}, {}
    for e, dt in enumerate((torch.bfloat16, torch.float16, torch.float32)):
        w = I.weights(48, 256, seed=20 + e)
        p, sc, _ = C.int4_pack_layer(w, 32, True)
        sc = (sc.float() * (1 + 2.0 ** -12)).to(dt) if dt != torch.bfloat16 else sc     # not bf16-representable
        name = f"model.layers.1.mlp.experts.{e}.down_proj"
        shard[f"{name}.weight_packed"], shard[f"{name}.weight_scale"] = p, sc
        shard[f"{name}.weight_shape"] = torch.tensor([48, 256], dtype=torch.int32)
        want[f"{name}.weight"] = C.int4_dequant_any(p, sc, (48, 256), 32)
    save_file(shard, str(src / "model.safetensors"))
    json.dump({"hidden_size": 256, "moe_intermediate_size": 48,
               "quantization_config": {"config_groups": {"group_0": {"weights": {"group_size": 32}}}}},
              open(src / "config.json", "w"))
    out = tmp_path / "bf16"
    K2.main(["--model-dir", str(src), "--output-dir", str(out)])
    got = load_file(str(out / "model.safetensors"))
    assert set(got) == set(want)
    for name, t in want.items():
        assert got[name].dtype == torch.bfloat16 and I.same_bits(got[name], t), name
