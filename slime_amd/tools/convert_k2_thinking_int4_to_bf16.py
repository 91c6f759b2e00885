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
import shutil
from collections import defaultdict

import torch
from safetensors import safe_open

from ..int4 import Int4DequantPlan, dequantize_int4
from . import _shards

_PROJECTIONS = ("gate_proj", "up_proj", "down_proj")
_SUFFIXES = ("weight_packed", "weight_scale", "weight_shape")


def _load_config(model_dir: str, config_path):
    """-> (hidden_size, moe_intermediate_size, group_size); group_size defaults to 128 (:38-52)."""
    with open(config_path or os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    group = cfg.get("quantization_config", {}).get("config_groups", {}).get("group_0", {}).get("weights", {})
    return int(cfg.get("hidden_size")), int(cfg.get("moe_intermediate_size")), int(group.get("group_size", 128))


def _dequantize_tensor(weight_packed, weight_scale, weight_shape, group_size: int) -> torch.Tensor:
    """Name and arguments of the reference function (:55-84); the arithmetic runs in ``wq_int4_dequant``."""
    if group_size <= 0:
        raise ValueError("per-channel scales (group_size <= 0) are not produced by the INT4 converters and not supported")
    if weight_scale.dtype != torch.bfloat16:
        raise TypeError(f"weight_scale must be bfloat16 (what pack-quantized checkpoints store), got {weight_scale.dtype}")
    return dequantize_int4(weight_packed.to(torch.int32), weight_scale, weight_shape, group_size)


def _is_quantized_weight_key(key: str) -> bool:
    """Routed (not shared) expert projections only (:87-96)."""
    if ".mlp.experts." not in key or ".shared_experts." in key:
        return False
    return any(key.endswith(f".{proj}.{suffix}") for proj in _PROJECTIONS for suffix in _SUFFIXES)


def convert_file(input_path: str, output_path: str, group_size: int, skip_existing: bool = True):
    if skip_existing and os.path.exists(output_path):
        return
    dev = _shards.device()
    tensors = {}
    experts = defaultdict(lambda: defaultdict(dict))
    for key, tensor in _shards.read_shard(input_path).items():
        parts = key.split(".")
        if not _is_quantized_weight_key(key) or "experts" not in parts:
            tensors[key] = tensor
            continue
        at = parts.index("experts")
        experts[".".join(parts[:at + 2])][parts[-2]][parts[-1]] = tensor
    names, packeds, scales, shapes = [], [], [], []
    for prefix, components in experts.items():
        for proj in _PROJECTIONS:
            data = components.get(proj, {})
            if not set(_SUFFIXES).issubset(data):
                for suffix, value in data.items():          # incomplete: stays quantized
                    tensors[f"{prefix}.{proj}.{suffix}"] = value
                continue
            if data["weight_scale"].dtype != torch.bfloat16:
                raise TypeError(f"{prefix}.{proj}.weight_scale must be bfloat16 (what pack-quantized checkpoints store), "
                                f"got {data['weight_scale'].dtype}")
            names.append(f"{prefix}.{proj}.weight")
            packeds.append(_shards.to_device(data["weight_packed"].to(torch.int32), dev))
            scales.append(_shards.to_device(data["weight_scale"], dev))
            shapes.append(data["weight_shape"])
    if names:
        if group_size <= 0 or group_size & (group_size - 1):
            # not a power of two: one kernel launch per tensor
            for name, p, sc, sh in zip(names, packeds, scales, shapes):
                tensors[name] = _dequantize_tensor(p, sc, sh, group_size).cpu()
        else:
            plan = Int4DequantPlan(packeds, scales, shapes, group_size)     # one launch and one copy for the shard
            plan.run()
            flat = plan.flat_y.cpu()
            base = plan.flat_y.data_ptr()
            for name, y in zip(names, plan.outputs):
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
    names = args.files if args.files else _shards.list_shards(model_dir)
    if not names:
        print("No safetensors checkpoints found.")
        return
    for name in names:
        path = os.path.join(model_dir, name)
        if os.path.isfile(path):
            print(f"Converting {name}")
            convert_file(path, os.path.join(output_dir, name), group_size, skip_existing=not args.overwrite)
    for fname in os.listdir(model_dir):
        if fname == "model.safetensors.index.json":
            continue
        if fname.endswith(".json") or fname.endswith(".py") or fname.startswith("tokenizer"):
            shutil.copy2(os.path.join(model_dir, fname), os.path.join(output_dir, fname))
    weight_map = {}
    for fname in _shards.list_shards(output_dir):
        with safe_open(os.path.join(output_dir, fname), framework="pt") as reader:
            for key in reader.keys():
                weight_map[key] = fname
    with open(os.path.join(output_dir, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f, indent=2)
    print(f"\nSuccessful! Output saved to: {output_dir}")


if __name__ == "__main__":
    main()
