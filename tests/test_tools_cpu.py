"""Key routing, config blocks and index quirks of the offline converters (CPU only)."""

import json

import torch

from slime_amd.tools import _shards
from slime_amd.tools import convert_hf_to_fp8 as F8
from slime_amd.tools import convert_hf_to_int4_direct as I4


def test_fp8_key_filter():
    conv = ["model.layers.0.self_attn.q_proj.weight", "model.layers.0.mlp.gate_proj.weight",
            "model.layers.0.mlp.experts.3.down_proj.weight", "model.layers.0.mlp.shared_experts.up_proj.weight"]
    keep = ["model.embed_tokens.weight", "lm_head.weight", "model.norm.weight", "model.layers.0.input_layernorm.weight",
            "model.layers.0.mlp.gate.weight", "model.layers.0.mlp.router.weight", "model.layers.0.self_attn.q_norm.weight",
            "model.layers.0.self_attn.q_proj.bias", "model.layers.0.linear_attn.conv1d.weight",
            "model.layers.0.linear_attn.A_log", "model.layers.0.linear_attn.in_proj_a.weight", "model.mtp.eh_proj.weight"]
    assert all(F8.is_converted(k) for k in conv)
    assert not any(F8.is_converted(k) for k in keep)
    assert F8.scale_name("a.b.weight", [128, 128]) == "a.b.weight_scale_inv"
    assert F8.scale_name("a.b.weight", None) == "a.b.weight_scale"


def test_fp8_config_blocks():
    cfg = F8.fp8_quantization_config("block", [128, 128], None, ["b", "a", "b"])
    assert cfg == {"activation_scheme": "dynamic", "fmt": "e4m3", "quant_method": "fp8", "weight_block_size": [128, 128],
                   "modules_to_not_convert": ["a", "b"]}
    assert F8.fp8_quantization_config("block", [128, 128], "ue8m0", [])["scale_fmt"] == "ue8m0"
    assert "weight_block_size" not in F8.fp8_quantization_config("tensor", None, "ue8m0", [])
    ch = F8.fp8_quantization_config("channel", None, None, ["x"])
    assert ch["format"] == "float-quantized" and ch["quant_method"] == "compressed-tensors" and ch["ignore"] == ["x"]
    assert ch["config_groups"]["group_0"]["weights"]["strategy"] == "channel"
    assert ch["config_groups"]["group_0"]["input_activations"]["strategy"] == "token"


def test_int4_rules_and_config():
    rules = I4.DEFAULT_IGNORE_RULES
    assert not I4.is_ignored("model.layers.1.mlp.experts.7.gate_proj.weight", rules)
    for n in ("lm_head.weight", "model.norm.weight", "model.embed_tokens.weight", "model.layers.1.self_attn.o_proj.weight",
              "model.layers.1.mlp.shared_experts.up_proj.weight", "model.layers.1.mlp.down_proj.weight",
              "model.layers.1.mlp.gate.weight"):
        assert I4.is_ignored(n, rules), n
    assert I4.is_ignored("abc.def", ["abc"]) and I4.is_ignored("abc", ["abc"]) and not I4.is_ignored("xabc", ["abc"])
    cfg = I4.int4_quantization_config(128, True, ["r"])
    assert cfg["format"] == "pack-quantized" and cfg["ignore"] == ["r"] and cfg["kv_cache_scheme"] is None
    w = cfg["config_groups"]["group_0"]["weights"]
    assert (w["group_size"], w["num_bits"], w["strategy"], w["symmetric"], w["type"]) == (128, 4, "group", True, "int")
    a = I4.parse_args(["--model-dir", "a", "--save-dir", "b"])
    assert a.group_size == 32 and a.is_symmetric is False and a.ignore_rules == rules and a.max_workers == 1


def test_index_total_size_is_sum_of_first_dims(tmp_path):
    r = _shards.ConversionResult()
    r.add_result("s1.safetensors", {"a": torch.zeros(7, 3), "b": torch.zeros(5)}, ["m"])
    r.add_result("s2.safetensors", {"c": torch.zeros(2, 9, 4)})
    assert r.param_count == 14 and r.modules_to_not_convert == ["m"]
    _shards.write_index(str(tmp_path), r)
    idx = json.load(open(tmp_path / "model.safetensors.index.json"))
    assert idx == {"weight_map": {"a": "s1.safetensors", "b": "s1.safetensors", "c": "s2.safetensors"},
                   "metadata": {"total_size": 14}}


def test_int4_to_bf16_key_rule():
    from slime_amd.tools import convert_k2_thinking_int4_to_bf16 as K2

    yes = ["model.layers.3.mlp.experts.17.gate_proj.weight_packed", "model.layers.3.mlp.experts.0.down_proj.weight_scale",
           "model.layers.60.mlp.experts.383.up_proj.weight_shape"]
    no = ["model.layers.3.mlp.shared_experts.gate_proj.weight_packed", "model.layers.3.mlp.experts.17.gate_proj.weight",
          "model.layers.3.self_attn.q_proj.weight_packed", "model.layers.3.mlp.experts.17.gate_proj.weight_zero_point",
          "model.layers.3.mlp.gate.weight"]
    assert all(K2._is_quantized_weight_key(k) for k in yes) and not any(K2._is_quantized_weight_key(k) for k in no)
    args = K2.parse_args(["--model-dir", "m", "--files", "a.safetensors", "b.safetensors", "--overwrite"])
    assert args.files == ["a.safetensors", "b.safetensors"] and args.overwrite and args.output_dir is None


def test_host_stage_bump_allocator_reuses_and_coalesces():
    """The staging area of the converters' device-to-host copies: aligned disjoint pieces, growth by chunks, one
    chunk of the combined size after the next shard begins, and no allocation from then on."""
    from slime_amd.tools._shards import _HostStage

    st = _HostStage()
    st.chunk_bytes = 4096
    a, b = st.take(1000), st.take(3500)          # second piece does not fit behind the first: new chunk
    c = st.take(10000)                           # bigger than a chunk
    assert [x.numel() for x in (a, b, c)] == [1000, 3500, 10000]
    assert len(st.chunks) == 3 and all(x.data_ptr() % 64 == 0 for x in (a, b, c))
    a.fill_(1), b.fill_(2), c.fill_(3)
    assert (int(a.sum()), int(b.sum()), int(c.sum())) == (1000, 7000, 30000)      # disjoint
    st.reset()
    assert len(st.chunks) == 1 and st.chunks[0].numel() == 4096 + 4096 + 10240
    base = st.chunks[0].data_ptr()
    pieces = [st.take(n) for n in (1000, 3500, 10000)]
    assert len(st.chunks) == 1 and pieces[0].data_ptr() == base
    assert pieces[1].data_ptr() == base + 1024 and pieces[2].data_ptr() == base + 1024 + 3584
    st.reset()
    assert st.take(0).numel() == 0 and st.take(5).data_ptr() == base + 256
