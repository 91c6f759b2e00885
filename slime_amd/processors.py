"""Quantise-on-update step of the Megatron -> rollout-engine weight sync.

Drop-in for slime/backends/megatron_utils/megatron_to_hf/processors/: same function names, arguments and
returned ``[(hf_name, tensor), ...]`` lists.

* ``quantize_params``                      - processors/__init__.py:6-22
* ``quantize_params_fp8`` / ``_quantize_param`` - processors/quantizer_fp8.py:10-118
* ``quantize_params_compressed_tensors``   - processors/quantizer_compressed_tensors.py:268-297

The UE8M0 (power-of-two scale) re-quantisation that the reference takes only when sglang's DeepGEMM
path is active (quantizer_fp8.py:103-108) does not exist on this hardware; ``transform_ue8m0`` is
accepted and ignored, as it is in the reference whenever that path is off.
"""

from __future__ import annotations

import re

import torch

from .fp8 import FP8_DTYPE, Fp8QuantPlan, blockwise_cast_to_fp8_triton, tensor_fp8
from .int4 import pack_layer

_LAYER_RE = re.compile(r"module\.module\.decoder\.layers\.(\d+)\.(.+)")
_MTP_LAYER_RE = re.compile(r"module\.module\.mtp\.layers\.(\d+)\.(.+)")
_EXPERT_RE = re.compile(r"mlp.experts\.(.+)\.weight(\d+)")
_SHARED_EXPERT_RE = re.compile(r"mlp.shared_experts\.(.+)")

# Megatron parameter names (below the layer prefix) whose HF tensors are quantised; quantizer_fp8.py:69-87
_DENSE_QUANTIZED = frozenset({
    "self_attention.linear_proj.weight",
    "self_attention.linear_qkv.weight",
    "mlp.linear_fc1.weight",
    "mlp.linear_fc2.weight",
    "self_attention.linear_q_proj.weight",
    "self_attention.linear_q_down_proj.weight",
    "self_attention.linear_q_up_proj.weight",
    "self_attention.linear_kv_down_proj.weight",
    "self_attention.linear_kv_up_proj.weight",
    "self_attention.wq_b.weight",
    "self_attention.wk.weight",
    "self_attention.linear_attn.in_proj_qkv.weight",
    "self_attention.linear_attn.in_proj_z.weight",
    "self_attention.linear_attn.out_proj.weight",
})


def _fp8_route(megatron_name: str):
    """-> None (pass through) | "all" | "skip_scales" (experts: drop entries named *_scale)."""
    m = _LAYER_RE.match(megatron_name)
    if m:
        rest = m.group(2)
    else:
        m = _MTP_LAYER_RE.match(megatron_name)
        if not m:
            return None
        rest = m.group(2).replace("transformer_layer.", "")
    m = _EXPERT_RE.match(rest)
    if m and m.group(1) in ("linear_fc1", "linear_fc2"):
        return "skip_scales"
    if m:
        rest = m.group(1)  # the reference rebinds `rest` on an expert match before the later checks
    m = _SHARED_EXPERT_RE.match(rest)
    if m and m.group(1) in ("linear_fc1.weight", "linear_fc2.weight"):
        return "all"
    if m:
        rest = m.group(1)
    return "all" if rest in _DENSE_QUANTIZED else None


def _quantize_param(name, weight, weight_block_size, transform_ue8m0=True):
    """-> [(name, qweight), (scale_name, scale)]; block scales are named ``.weight_scale_inv``, per-tensor
    scales ``.weight_scale`` (quantizer_fp8.py:98-118)."""
    assert name.endswith(".weight"), f"Expected weight parameter, got {name}"
    if weight_block_size is not None:
        qweight, scale = blockwise_cast_to_fp8_triton(weight, weight_block_size)
        scale_name = name.replace(".weight", ".weight_scale_inv")
    else:
        qweight, scale = tensor_fp8(weight)
        scale_name = name.replace(".weight", ".weight_scale")
    return [(name, qweight), (scale_name, scale)]


def quantize_params_fp8(args, megatron_name, converted_named_params, quantization_config, transform_ue8m0=True):
    assert quantization_config["quant_method"] == "fp8"
    fmt = quantization_config.get("fmt", "e4m3")
    assert fmt == "e4m3", f"Unsupported FP8 format: {fmt}"
    assert quantization_config["activation_scheme"] == "dynamic"
    weight_block_size = quantization_config.get("weight_block_size", None)

    route = _fp8_route(megatron_name)
    if route is None:
        return converted_named_params
    todo = [(n, p) for n, p in converted_named_params if not (route == "skip_scales" and n.endswith("_scale"))]
    for n, _ in todo:
        assert n.endswith(".weight"), f"Expected weight parameter, got {n}"

    # q/k/v or gate/up of one Megatron parameter: one grouped launch instead of one launch per tensor
    if weight_block_size is not None and len(todo) > 1 and all(
            p.is_cuda and p.dim() == 2 and p.dtype == torch.bfloat16 for _, p in todo):
        outs = Fp8QuantPlan([p for _, p in todo], weight_block_size, mode=1).run()
        result = []
        for (n, _), (q, s) in zip(todo, outs):
            result += [(n, q), (n.replace(".weight", ".weight_scale_inv"), s)]
        return result

    result = []
    for n, p in todo:
        result.extend(_quantize_param(n, p, weight_block_size, transform_ue8m0))
    return result


def _is_ignored(name: str, ignore_rules) -> bool:
    """``re:<regex>`` rules use re.match, others match exactly or as a prefix
    (quantizer_compressed_tensors.py:277-279)."""
    for rule in ignore_rules:
        if rule.startswith("re:"):
            if re.match(rule[3:], name):
                return True
        elif rule == name or name.startswith(rule):
            return True
    return False


def quantize_params_compressed_tensors(converted_named_params, quantization_config):
    w_cfg = quantization_config["config_groups"]["group_0"]["weights"]
    group_size = w_cfg["group_size"]
    is_symmetric = w_cfg["symmetric"]
    ignore_rules = quantization_config.get("ignore", [])

    results = []
    for name, param in converted_named_params:
        if _is_ignored(name, ignore_rules) or not name.endswith(".weight") or param.dim() < 2:
            results.append((name, param))
            continue
        packed, scale, zero_point = pack_layer(param, group_size, is_symmetric)
        if zero_point is not None:
            results.append((name.replace(".weight", ".weight_zero_point"), zero_point))
        results.append((name.replace(".weight", ".weight_packed"), packed))
        results.append((name.replace(".weight", ".weight_scale"), scale))
        results.append((name.replace(".weight", ".weight_shape"),
                        torch.tensor(param.shape, dtype=torch.int32, device=param.device)))
    return results


def quantize_params(args, megatron_name, converted_named_params, quantization_config, transform_ue8m0=True):
    """Dispatch on ``quantization_config["quant_method"]``; ``None`` config and unknown methods pass the
    parameters through unchanged (processors/__init__.py:6-22)."""
    if quantization_config is None:
        return converted_named_params
    method = quantization_config["quant_method"]
    if method == "fp8":
        return quantize_params_fp8(args, megatron_name, converted_named_params, quantization_config, transform_ue8m0)
    if method == "compressed-tensors":
        return quantize_params_compressed_tensors(converted_named_params, quantization_config)
    return converted_named_params


__all__ = ["quantize_params", "quantize_params_fp8", "_quantize_param", "quantize_params_compressed_tensors",
           "FP8_DTYPE"]
