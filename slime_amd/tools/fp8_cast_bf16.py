"""block-FP8 HF checkpoint -> bf16 HF checkpoint (command line and file formats of tools/fp8_cast_bf16.py).

python -m slime_amd.tools.fp8_cast_bf16 --input-fp8-hf-path IN --output-bf16-hf-path OUT

Per shard: every one-byte tensor whose ``<name>_scale_inv`` exists anywhere in the checkpoint is dequantised
(all of them by ONE grouped launch); ``*_scale_inv`` tensors are dropped from the shards and from the index;
a one-byte tensor without a scale is kept as it is, with a warning, as the reference does (:87-89).
"""

from __future__ import annotations

import glob
import json
import os
import shutil
from argparse import ArgumentParser

import torch

from ..fp8 import Fp8DequantPlan
from . import _shards

_SIDE_PATTERNS = ("config.json", "*.py", "tokenizer*", "chat_template*")   # what the reference copies with cp -rf


def main(fp8_path, bf16_path, block_size: int = 128):
    dev = _shards.device()
    os.makedirs(bf16_path, exist_ok=True)
    for pat in _SIDE_PATTERNS:
        for src in glob.glob(os.path.join(fp8_path, pat)):
            dst = os.path.join(bf16_path, os.path.basename(src))
            if os.path.isdir(src):
                shutil.copytree(src, dst, dirs_exist_ok=True)
            else:
                shutil.copyfile(src, dst)
    with open(os.path.join(fp8_path, "model.safetensors.index.json")) as f:
        weight_map = json.load(f)["weight_map"]

    cache = {}      # file name -> {tensor name: CPU tensor}; the two most recently used shards stay open

    def shard(name):
        if name not in cache:
            cache[name] = _shards.read_shard(os.path.join(fp8_path, name))
        return cache[name]

    dequantized = []
    for path in sorted(glob.glob(os.path.join(fp8_path, "*.safetensors"))):
        file_name = os.path.basename(path)
        print(f"Handling file: {path}")
        _shards.begin_shard()
        current = shard(file_name)
        out, codes, scales, names = {}, [], [], []
        for name, t in current.items():
            if name.endswith("_scale_inv"):
                continue
            if t.element_size() == 1:
                sname = f"{name}_scale_inv"
                if sname in weight_map:
                    names.append(name)
                    codes.append(_shards.to_device(t.view(torch.float8_e4m3fn), dev).contiguous())
                    scales.append(_shards.to_device(shard(weight_map[sname])[sname], dev).contiguous())
                    out[name] = None
                    continue
                print(f"Warning: Missing scale_inv tensor for {name}, skipping conversion")
            out[name] = t
        if names:
            plan = Fp8DequantPlan(codes, scales, block_size, 0, torch.bfloat16)
            plan.run()
            flat = _shards.to_host(plan.flat_y)        # one copy for the whole shard
            base = plan.flat_y.data_ptr()
            for name, y in zip(names, plan.outputs):
                off = (y.data_ptr() - base) // 2
                out[name] = flat[off:off + y.numel()].view(y.shape)
            dequantized.extend(names)
        _shards.write_shard(out, os.path.join(bf16_path, file_name), with_format_tag=False)
        while len(cache) > 2:
            del cache[next(iter(cache))]

    for name in dequantized:
        weight_map.pop(f"{name}_scale_inv", None)
    with open(os.path.join(bf16_path, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f, indent=2)


if __name__ == "__main__":
    parser = ArgumentParser()
    parser.add_argument("--input-fp8-hf-path", type=str, required=True)
    parser.add_argument("--output-bf16-hf-path", type=str, required=True)
    args = parser.parse_args()
    main(args.input_fp8_hf_path, args.output_bf16_hf_path)
