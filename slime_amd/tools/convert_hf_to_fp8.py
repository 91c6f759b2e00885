"""bf16 HF checkpoint -> FP8 HF checkpoint (command line and file formats of tools/convert_hf_to_fp8.py).

python -m slime_amd.tools.convert_hf_to_fp8 --model-dir IN --save-dir OUT [--strategy {block,channel,tensor}]
        [--block-size BM BN] [--max-workers N] [--scale-fmt ue8m0]

Per shard: the tensors selected for conversion go to the GPU, all block-quantised weights of the shard are
produced by ONE grouped launch into a flat buffer, and the results come back as two device-to-host copies.
"""

from __future__ import annotations

import argparse
import gc
import os
import sys
from concurrent.futures import ThreadPoolExecutor

import torch

from .. import arith
from ..fp8 import Fp8QuantPlan, block_fp8, channel_fp8, tensor_fp8
from . import _shards

# substrings that keep a "weight" tensor in its original dtype (tools/convert_hf_to_fp8.py:134-149)
_KEEP_SUBSTRINGS = ("layernorm", "embed", "router", "mlp.gate.", "norm", "lm_head", "eh_proj", "weights_proj",
                    "conv1d", "A_log", "dt_bias", "in_proj_a", "in_proj_b")


def is_converted(key: str) -> bool:
    return "weight" in key and not any(s in key for s in _KEEP_SUBSTRINGS)


def scale_name(key: str, block_size) -> str:
    return key.replace(".weight", ".weight_scale_inv" if block_size else ".weight_scale")


def fp8_quantization_config(strategy: str, block_size, scale_fmt, modules_to_not_convert) -> dict:
    """config.json "quantization_config" (tools/convert_hf_to_fp8.py:189-238).  The reference de-duplicates the
    skipped module names through a set, which leaves their order arbitrary; they are sorted here."""
    skipped = sorted(set(modules_to_not_convert))
    if strategy in ("block", "tensor"):
        cfg = {"activation_scheme": "dynamic", "fmt": "e4m3", "quant_method": "fp8"}
        if block_size:
            cfg["weight_block_size"] = block_size
            if scale_fmt is not None:
                cfg["scale_fmt"] = scale_fmt
        if skipped:
            cfg["modules_to_not_convert"] = skipped
        return cfg
    activations = {"actorder": None, "block_structure": None, "dynamic": True, "group_size": None, "num_bits": 8,
                   "observer": None, "observer_kwargs": {}, "strategy": "token", "symmetric": True, "type": "float"}
    weights = {"actorder": None, "block_structure": None, "dynamic": False, "group_size": None, "num_bits": 8,
               "observer": "minmax", "observer_kwargs": {}, "strategy": strategy, "symmetric": True, "type": "float"}
    group = {"group_0": {"input_activations": activations, "output_activations": None, "targets": ["Linear"],
                         "weights": weights}}
    return {"config_groups": group, "format": "float-quantized", "ignore": skipped,
            "quant_method": "compressed-tensors", "quantization_status": "compressed"}


def process_file(input_path, output_path, filename, strategy, block_size, result_collector, arithmetic=None):
    """``arithmetic``: the torch evaluation ("device" / "cpu") the caller resolved once; worker threads do not see the
    caller's thread-local choice, so it travels as an argument."""
    if not filename.endswith(".safetensors"):
        return
    with arith.torch_arithmetic(arithmetic or arith.get_torch_arithmetic()):
        _process_file(input_path, output_path, filename, strategy, block_size, result_collector)


def _process_file(input_path, output_path, filename, strategy, block_size, result_collector):
    dev = _shards.device()
    _shards.begin_shard()
    weights = _shards.read_shard(os.path.join(input_path, filename))
    out, skipped = {}, []
    todo = [k for k in weights if is_converted(k)]
    for k in weights:
        if k not in todo:
            skipped.append(k.replace(".weight", ""))
            out[k] = weights[k]
    if todo:
        on_gpu = [_shards.to_device(weights[k], dev) for k in todo]
        if strategy not in ("tensor", "channel"):
            # bf16 matrices (what checkpoints hold) share one launch; other float dtypes, which block_fp8 also takes,
            # go one by one through the kernel with that dtype's arithmetic
            planned = [i for i, w in enumerate(on_gpu) if w.dtype == torch.bfloat16 and w.dim() == 2]
            for i, (k, w) in enumerate(zip(todo, on_gpu)):
                if i not in planned:
                    out[k], out[scale_name(k, block_size)] = _shards.to_host(*block_fp8(w, block_size))
            if planned:
                plan = Fp8QuantPlan([on_gpu[i] for i in planned], block_size)
                plan.run()
                flat_q, flat_s = _shards.to_host(plan.flat_q, plan.flat_s)     # two copies for the whole shard
                qbase, sbase = plan.flat_q.data_ptr(), plan.flat_s.data_ptr()
                for i, (q, s) in zip(planned, plan.outputs):
                    k = todo[i]
                    qo = q.data_ptr() - qbase
                    so = (s.data_ptr() - sbase) // 4
                    out[k] = flat_q[qo:qo + q.numel()].view(torch.float8_e4m3fn).view(q.shape)
                    out[scale_name(k, block_size)] = flat_s[so:so + s.numel()].view(s.shape)
        else:
            fn = tensor_fp8 if strategy == "tensor" else channel_fp8
            for k, w in zip(todo, on_gpu):
                out[k], out[scale_name(k, block_size)] = _shards.to_host(*fn(w))
    # keep the reference's key order: converted weight followed by its scale, in shard order
    ordered = {}
    for k in weights:
        ordered[k] = out[k]
        if k in todo:
            ordered[scale_name(k, block_size)] = out[scale_name(k, block_size)]
    _shards.write_shard(ordered, os.path.join(output_path, filename))
    result_collector.add_result(filename, ordered, skipped)


def convert_fp8(input_path, output_path, strategy, block_size=None, max_workers=4, scale_fmt=None):
    input_path = os.path.abspath(input_path)
    os.makedirs(output_path, exist_ok=True)
    _shards.copy_side_files(input_path, output_path)
    result = _shards.ConversionResult()
    if scale_fmt is not None:
        # exactly what the reference tool does with the flag (tools/convert_hf_to_fp8.py:197-198): the key goes into
        # config.json and the arithmetic stays block_fp8's - the scales written are NOT powers of two
        print(f"convert_hf_to_fp8: --scale-fmt {scale_fmt} only records \"scale_fmt\" in config.json, as the reference "
              "tool does; the weight_scale_inv tensors keep ordinary float32 scales (power-of-two scales: "
              "slime_amd.quant_weight_ue8m0)", file=sys.stderr)
    arithmetic = arith.get_torch_arithmetic()        # resolved once, on the calling thread
    with ThreadPoolExecutor(max_workers=max_workers) as pool:
        futures = [pool.submit(process_file, input_path, output_path, f, strategy, block_size, result, arithmetic)
                   for f in _shards.list_shards(input_path)]
        for fut in futures:
            fut.result()
    _shards.write_config(input_path, output_path,
                         fp8_quantization_config(strategy, block_size, scale_fmt, result.modules_to_not_convert))
    _shards.write_index(output_path, result)
    gc.collect()
    torch.cuda.empty_cache()


def main(argv=None):
    parser = argparse.ArgumentParser()
    parser.add_argument("--model-dir", type=str, help="Path to the directory of the HF safetensors model.")
    parser.add_argument("--save-dir", type=str, help="Path to the directory to save the converted model.")
    parser.add_argument("--strategy", type=str, default="block", choices=["block", "channel", "tensor"])
    parser.add_argument("--block-size", type=int, nargs="*", default=None, help="eg. --block-size 128 128")
    parser.add_argument("--max-workers", type=int, default=1, help="Number of worker threads for parallel processing")
    parser.add_argument("--scale-fmt", type=str, default=None, choices=["ue8m0"])
    args = parser.parse_args(argv)
    if not os.path.exists(args.save_dir):
        print(f"Creating directory {args.save_dir}")
        os.makedirs(args.save_dir)
    elif not os.path.isdir(args.save_dir):
        raise ValueError("The save_dir should be a directory.")
    convert_fp8(args.model_dir, args.save_dir, args.strategy, args.block_size, args.max_workers, args.scale_fmt)


if __name__ == "__main__":
    main()
