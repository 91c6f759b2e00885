"""SafetensorReader: the reference's own reader tests (tests/test_hf_to_megatron.py:345-358,
tests/test_qwen3_5_vl_native.py:194-202) plus the layouts a real checkpoint has."""

import json

import pytest
import torch
from safetensors.torch import save_file

from oracle import c_oracle as C
from slime_amd import SafetensorReader
from tests import wq_inputs as I

E4M3 = torch.float8_e4m3fn


def test_safetensor_reader_caches_only_the_last_tensor(tmp_path):
    save_file({"first": torch.ones(2), "second": torch.zeros(2)}, tmp_path / "model.safetensors")
    reader = SafetensorReader(tmp_path)

    first = reader.get_tensor("first")
    assert reader.get_tensor("first") is first
    reader.get_tensor("second")
    assert reader.get_tensor("first") is not first


def test_reader_lookup_rules(tmp_path):
    with pytest.raises(FileNotFoundError):
        SafetensorReader(tmp_path)
    save_file({"a.weight": torch.arange(6.0).view(2, 3)}, tmp_path / "model-00001-of-00002.safetensors")
    save_file({"b.weight": torch.ones(4, dtype=torch.bfloat16), "c": torch.zeros(3, dtype=torch.uint8)},
              tmp_path / "model-00002-of-00002.safetensors")
    reader = SafetensorReader(tmp_path)                       # no index: the files are scanned
    assert "a.weight" in reader and "b.weight" in reader and "zzz" not in reader
    assert torch.equal(reader.get_tensor("a.weight"), torch.arange(6.0).view(2, 3))
    assert reader.get_tensor("b.weight").dtype == torch.bfloat16
    assert reader.get_tensor("c").dtype == torch.uint8       # one byte per element but no scale: returned as stored
    with pytest.raises(KeyError, match="does not contain 'zzz'"):
        reader.get_tensor("zzz")
    json.dump({"weight_map": {"a.weight": "model-00001-of-00002.safetensors"}}, open(tmp_path / "model.safetensors.index.json", "w"))
    assert "b.weight" not in SafetensorReader(tmp_path)      # with an index, the index decides


@pytest.mark.gpu
def test_reader_dequantizes_block_scaled_fp8(tmp_path, cuda):
    weight = torch.linspace(-2, 2, 128 * 128).view(128, 128).to(E4M3)
    scale = torch.tensor([[2.0]])
    save_file({"weight": weight, "weight_scale_inv": scale}, tmp_path / "model.safetensors")

    loaded = SafetensorReader(tmp_path).get_tensor("weight")

    assert loaded.dtype == torch.bfloat16 and loaded.device.type == "cpu"          # host tensors, like the reference's reader
    assert torch.equal(loaded, weight.to(torch.bfloat16) * 2)
    on_gpu = SafetensorReader(tmp_path, device="cuda").get_tensor("weight")
    assert on_gpu.is_cuda and torch.equal(on_gpu.cpu(), loaded)


@pytest.mark.gpu
def test_reader_partly_quantised_checkpoint_and_other_one_byte_dtypes(tmp_path, cuda):
    """modules_to_not_convert leaves bf16 weights next to FP8 ones: both come back on the host and can be concatenated.
    A one-byte tensor that is not float8_e4m3fn is not reinterpreted: without a scale it is returned as stored, with a
    scale it is refused."""
    codes = I.fp8_codes(128, 256, seed=3)
    scale = I.log_uniform_scales(1, 2, seed=4)
    save_file({"q.weight": codes.view(E4M3), "q.weight_scale_inv": scale, "k.weight": torch.ones(64, 256, dtype=torch.bfloat16),
               "flags": torch.arange(5, dtype=torch.int8), "odd.weight": torch.zeros(128, 128, dtype=torch.int8),
               "odd.weight_scale_inv": torch.ones(1, 1)}, tmp_path / "model.safetensors")
    reader = SafetensorReader(tmp_path)
    qk = torch.cat([reader.get_tensor("q.weight"), reader.get_tensor("k.weight")], dim=0)
    assert qk.shape == (192, 256) and I.same_bits(qk[:128], C.fp8_block_dequant(codes, scale, 128, 1))
    assert reader.get_tensor("flags").dtype == torch.int8
    with pytest.raises(TypeError, match="float8_e4m3fn"):
        reader.get_tensor("odd.weight")


@pytest.mark.gpu
def test_reader_ragged_shapes_and_scale_in_another_shard(tmp_path, cuda):
    shapes = {"l0.q_proj.weight": (300, 200), "l0.down_proj.weight": (7, 520), "l1.up_proj.weight": (256, 384)}
    first, second, want = {}, {}, {}
    for k, (name, (m, n)) in enumerate(shapes.items()):
        codes = I.fp8_codes(m, n, seed=k)
        scale = I.log_uniform_scales(-(-m // 128), -(-n // 128), seed=10 + k)
        first[name] = codes.view(E4M3)
        second[name + "_scale_inv"] = scale                   # every scale lives in the other shard
        want[name] = C.fp8_block_dequant(codes, scale, 128, 1)
    first["l0.norm.weight"] = torch.ones(8, dtype=torch.bfloat16)
    save_file(first, tmp_path / "model-00001-of-00002.safetensors")
    save_file(second, tmp_path / "model-00002-of-00002.safetensors")
    reader = SafetensorReader(tmp_path, device="cuda")
    for name, w in want.items():
        got = reader.get_tensor(name)
        assert got.is_cuda and got.dtype == torch.bfloat16 and got.shape == w.shape and I.same_bits(got.cpu(), w), name
        # the reference's op sequence on the host: pad, view as blocks, multiply by the bf16 scale in place
        m, n = w.shape
        s = second[name + "_scale_inv"].to(torch.bfloat16)
        t = torch.nn.functional.pad(first[name].to(torch.bfloat16), (0, s.shape[1] * 128 - n, 0, s.shape[0] * 128 - m))
        t = t.view(s.shape[0], 128, s.shape[1], 128)
        t.mul_(s[:, None, :, None])
        assert I.same_bits(got.cpu(), t.reshape(s.shape[0] * 128, s.shape[1] * 128)[:m, :n].contiguous()), name
    assert reader.get_tensor("l0.norm.weight").dtype == torch.bfloat16 and not reader.get_tensor("l0.norm.weight").is_cuda
    assert reader.get_tensor("l0.q_proj.weight_scale_inv").dtype == torch.float32     # a scale asked for by name: as stored
