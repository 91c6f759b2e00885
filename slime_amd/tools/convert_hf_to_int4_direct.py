"""bf16 HF checkpoint -> INT4 (compressed-tensors pack-quantized) HF checkpoint, round-to-nearest
(command line and file formats of tools/convert_hf_to_int4_direct.py).

python -m slime_amd.tools.convert_hf_to_int4_direct --model-dir IN --save-dir OUT [--group-size G] [--is-symmetric]
        [--ignore-rules RULE ...] [--max-workers N]

Per shard: all symmetric-quantised weights are produced by ONE grouped launch (groups of 32 / 64 / 128); other
group sizes and the asymmetric form go tensor by tensor through ``pack_layer``.
"""

from __future__ import annotations

import argparse
import gc
import os
import re
from concurrent.futures import ThreadPoolExecutor

import torch

from ..int4 import Int4PackPlan, pack_layer
from . import _shards

DEFAULT_IGNORE_RULES = ["re:.*lm_head.*", "re:.*norm.*", "re:.*embed.*", "re:.*self_attn.*", "re:.*shared_experts.*",
                        "re:.*mlp\\.(gate|up|gate_up|down)_proj.*", "re:.*mlp\\.gate\\.*"]


def is_ignored(name: str, ignore_rules) -> bool:
    """``re:<regex>`` rules use re.match; other rules match exactly or as a prefix (:181-184)."""
    for rule in ignore_rules:
        if rule.startswith("re:"):
            if re.match(rule[3:], name):
                return True
        elif rule == name or name.startswith(rule):
            return True
    return False


def int4_quantization_config(group_size: int, is_symmetric: bool, ignore_rules) -> dict:
    weights = {"actorder": None, "block_structure": None, "dynamic": False, "group_size": group_size, "num_bits": 4,
               "observer": "minmax", "observer_kwargs": {}, "strategy": "group", "symmetric": is_symmetric,
               "type": "int"}
    group = {"group_0": {"input_activations": None, "output_activations": None, "targets": ["Linear"],
                         "weights": weights}}
    return {"config_groups": group, "format": "pack-quantized", "ignore": ignore_rules, "kv_cache_scheme": None,
            "quant_method": "compressed-tensors", "quantization_status": "compressed"}


def process_file(input_path, output_path, filename, group_size, is_symmetric, ignore_rules, result_collector):
    dev = _shards.device()
    _shards.begin_shard()
    weights = _shards.read_shard(os.path.join(input_path, filename))
    todo = [n for n, w in weights.items()
            if not is_ignored(n, ignore_rules) and n.endswith(".weight") and w.dim() >= 2]
    results = {}
    if todo:
        on_gpu = [_shards.to_device(weights[n], dev) for n in todo]
        fused = is_symmetric and group_size in (32, 64, 128) and all(
            w.dim() == 2 and w.dtype == torch.bfloat16 and w.shape[1] % group_size == 0 for w in on_gpu)
        if fused:
            plan = Int4PackPlan([w.contiguous() for w in on_gpu], group_size)
            plan.run()
            flat_p, flat_s = _shards.to_host(plan.flat_packed, plan.flat_scale)
            pbase, sbase = plan.flat_packed.data_ptr(), plan.flat_scale.data_ptr()
            for n, (p, s) in zip(todo, plan.outputs):
                po, so = (p.data_ptr() - pbase) // 4, (s.data_ptr() - sbase) // 2
                results[n] = (flat_p[po:po + p.numel()].view(p.shape), flat_s[so:so + s.numel()].view(s.shape), None)
        else:
            for n, w in zip(todo, on_gpu):
                p, s, zp = pack_layer(w, group_size, is_symmetric)
                results[n] = (*_shards.to_host(p, s), None if zp is None else _shards.to_host(zp))
    out = {}
    for n, w in weights.items():
        if n not in results:
            out[n] = w
            continue
        p, s, zp = results[n]
        if zp is not None:
            out[n.replace(".weight", ".weight_zero_point")] = zp
        out[n.replace(".weight", ".weight_packed")] = p
        out[n.replace(".weight", ".weight_scale")] = s
        out[n.replace(".weight", ".weight_shape")] = torch.tensor(w.shape, dtype=torch.int32)
    _shards.write_shard(out, os.path.join(output_path, filename))
    result_collector.add_result(filename, out)


def convert_int4(input_path, output_path, group_size, is_symmetric, ignore_rules, max_workers):
    input_path = os.path.abspath(input_path)
    os.makedirs(output_path, exist_ok=True)
    _shards.copy_side_files(input_path, output_path)
    result = _shards.ConversionResult()
    with ThreadPoolExecutor(max_workers=max_workers) as pool:
        futures = [pool.submit(process_file, input_path, output_path, f, group_size, is_symmetric, ignore_rules, result)
                   for f in _shards.list_shards(input_path)]
        for fut in futures:
            fut.result()
    _shards.write_config(input_path, output_path, int4_quantization_config(group_size, is_symmetric, ignore_rules))
    _shards.write_index(output_path, result)
    gc.collect()
    torch.cuda.empty_cache()
    return output_path


def parse_args(argv=None):
    parser = argparse.ArgumentParser()
    parser.add_argument("--model-dir", type=str, required=True, help="local BF16 path")
    parser.add_argument("--save-dir", type=str, required=True)
    parser.add_argument("--group-size", type=int, default=32, help="Group Size")
    parser.add_argument("--is-symmetric", action="store_true", help="Whether to use symmetric quantization")
    parser.add_argument("--ignore-rules", nargs="+", default=list(DEFAULT_IGNORE_RULES), help="Ignore Rules")
    parser.add_argument("--max-workers", type=int, default=1, help="Number of worker threads for parallel processing")
    return parser.parse_args(argv)


def main(argv=None):
    args = parse_args(argv)
    if not os.path.exists(args.save_dir):
        print(f"Creating directory {args.save_dir}")
        os.makedirs(args.save_dir)
    elif not os.path.isdir(args.save_dir):
        raise ValueError("The save_dir should be a directory.")
    convert_int4(args.model_dir, args.save_dir, args.group_size, args.is_symmetric, args.ignore_rules, args.max_workers)
    print(f"Conversion complete, output saved to {args.save_dir}")


if __name__ == "__main__":
    main()
