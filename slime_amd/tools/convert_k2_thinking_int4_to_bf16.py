"""INT4 (pack-quantized MoE experts) HF checkpoint -> bf16 HF checkpoint: command line, key rules and output files
of tools/convert_k2_thinking_int4_to_bf16.py.

python -m slime_amd.tools.convert_k2_thinking_int4_to_bf16 --model-dir IN [--output-dir OUT] [--files F ...]
                                                            [--config-path CONFIG] [--overwrite]

Per shard: every routed expert's gate/up/down projection that has all three of ``weight_packed``, ``weight_scale``
and ``weight_shape`` becomes one bf16 ``weight`` (HIP kernel); incomplete triples and every other tensor are kept as
they are.  ``*.json`` / ``*.py`` / ``tokenizer*`` files are copied and a fresh index is written with empty metadata,
as the reference does (:214-237).
"""

from __future__ import annotations

import argparse
import json
import os
import re

import torch

from ..int4 import Int4DequantPlan, dequantize_int4
from . import _shards

# <prefix>.mlp.experts.<e>.<proj>.<part> of a routed (not shared) expert
_EXPERT_KEY = re.compile(r"^(?P<module>.*\.mlp\.experts\.[^.]+\.(?:gate_proj|up_proj|down_proj))"
                         r"\.(?P<part>weight_packed|weight_scale|weight_shape)$")
_PARTS = ("weight_packed", "weight_scale", "weight_shape")


def _load_config(model_dir: str, config_path):
    """-> (hidden_size, moe_intermediate_size, group_size); group_size defaults to 128 (:38-52)."""
    with open(config_path or os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    group = cfg.get("quantization_config", {}).get("config_groups", {}).get("group_0", {}).get("weights", {})
    return int(cfg.get("hidden_size")), int(cfg.get("moe_intermediate_size")), int(group.get("group_size", 128))


def _dequantize_tensor(weight_packed, weight_scale, weight_shape, group_size: int) -> torch.Tensor:
    """Name and arguments of the reference function (:55-84), any scale dtype and ``group_size <= 0`` included; the
    arithmetic runs in the HIP kernels behind ``dequantize_int4``."""
    return dequantize_int4(weight_packed.to(torch.int32), weight_scale, weight_shape, group_size)


def _is_quantized_weight_key(key: str) -> bool:
    """Routed (not shared) expert projections only (:87-96)."""
    return ".shared_experts." not in key and _EXPERT_KEY.match(key) is not None


def convert_file(input_path: str, output_path: str, group_size: int, skip_existing: bool = True):
    if skip_existing and os.path.exists(output_path):
        return
    dev = _shards.device()
    _shards.begin_shard()
    shard = _shards.read_shard(input_path)
    modules = {}                                  # module name -> {part: tensor}, in shard order
    for key, tensor in shard.items():
        m = _EXPERT_KEY.match(key) if _is_quantized_weight_key(key) else None
        if m:
            modules.setdefault(m["module"], {})[m["part"]] = tensor
    complete = {name: parts for name, parts in modules.items() if all(p in parts for p in _PARTS)}
    # everything that is not part of a complete triple is kept as it is (an incomplete triple stays quantized)
    tensors = {key: t for key, t in shard.items()
               if not (_is_quantized_weight_key(key) and _EXPERT_KEY.match(key)["module"] in complete)}
    one_launch = group_size > 0 and group_size & (group_size - 1) == 0 and group_size >= 8
    bucket = []
    for name, parts in complete.items():
        packed = _shards.to_device(parts["weight_packed"].to(torch.int32), dev)
        scale = _shards.to_device(parts["weight_scale"], dev)
        if one_launch and scale.dtype == torch.bfloat16:
            bucket.append((f"{name}.weight", packed, scale, parts["weight_shape"]))
        else:       # fp16 / fp32 scales, per-element scales, odd group sizes: one launch per tensor
            tensors[f"{name}.weight"] = _shards.to_host(_dequantize_tensor(packed, scale, parts["weight_shape"], group_size))
    if bucket:
        plan = Int4DequantPlan([b[1] for b in bucket], [b[2] for b in bucket], [b[3] for b in bucket], group_size)
        plan.run()                                # one launch and one copy for the shard
        flat, base = _shards.to_host(plan.flat_y), plan.flat_y.data_ptr()
        for (name, *_), y in zip(bucket, plan.outputs):
            off = (y.data_ptr() - base) // 2
            tensors[name] = flat[off:off + y.numel()].view(y.shape)
    os.makedirs(os.path.dirname(output_path), exist_ok=True)
    _shards.write_shard(tensors, output_path, with_format_tag=False)


def parse_args(argv=None) -> argparse.Namespace:
    parser = argparse.ArgumentParser(description="Convert GPTQ MoE experts to BF16 weights.")
    parser.add_argument("--model-dir", required=True, help="Directory containing safetensors checkpoints.")
    parser.add_argument("--output-dir", default=None, help="Destination BF16 model directory (default: <model-dir>_bf16).")
    parser.add_argument("--files", nargs="+", default=None, help="Optional specific safetensor files to convert.")
    parser.add_argument("--config-path", default=None, help="Path to config.json if not in model-dir.")
    parser.add_argument("--overwrite", action="store_true", help="Overwrite existing BF16 files.")
    return parser.parse_args(argv)


def main(argv=None):
    args = parse_args(argv)
    model_dir = os.path.abspath(args.model_dir)
    output_dir = os.path.abspath(args.output_dir or f"{model_dir}_bf16")
    if not os.path.isdir(model_dir):
        raise FileNotFoundError(f"Model directory not found: {model_dir}")
    _, _, group_size = _load_config(model_dir, args.config_path)
    shards = [n for n in (args.files or _shards.list_shards(model_dir)) if os.path.isfile(os.path.join(model_dir, n))]
    if not (args.files or shards):
        print("No safetensors checkpoints found.")
        return
    for name in shards:
        print(f"Converting {name}")
        convert_file(os.path.join(model_dir, name), os.path.join(output_dir, name), group_size,
                     skip_existing=not args.overwrite)
    os.makedirs(output_dir, exist_ok=True)
    _shards.copy_matching_files(model_dir, output_dir, skip=("model.safetensors.index.json",),
                                keep=lambda n: n.endswith((".json", ".py")) or n.startswith("tokenizer"))
    _shards.write_index_of_directory(output_dir)
    print(f"\nSuccessful! Output saved to: {output_dir}")


if __name__ == "__main__":
    main()
