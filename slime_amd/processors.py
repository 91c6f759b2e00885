"""Quantise-on-update step of the Megatron -> rollout-engine weight sync.

Drop-in for slime/backends/megatron_utils/megatron_to_hf/processors/: same function names, arguments and
returned ``[(hf_name, tensor), ...]`` lists.

* ``quantize_params``                      - processors/__init__.py:6-22
* ``quantize_params_fp8`` / ``_quantize_param`` - processors/quantizer_fp8.py:10-118
* ``quantize_params_compressed_tensors``   - processors/quantizer_compressed_tensors.py:268-297

The UE8M0 (power-of-two scale) re-quantisation, which the reference takes only when sglang reports a DeepGEMM rollout
engine (quantizer_fp8.py:103-108), is off unless ``set_ue8m0_requant(True)`` switches it on; then ``_quantize_param``
returns power-of-two float32 scales, and ``transform_ue8m0=True`` - the repacking into DeepGEMM's TMA layout - raises
``NotImplementedError`` instead of being ignored.  With the switch off ``transform_ue8m0`` has no effect, exactly as in
the reference whenever that path is off.
"""

from __future__ import annotations

import ctypes
import re
import threading
from collections import OrderedDict

import numpy as np
import torch

from . import _lib
from ._tables import ResolvedTable
from .fp8 import (FP8_DTYPE, blockwise_cast_to_fp8_triton, ceildiv, quant_weight_ue8m0, tensor_fp8, tile_table,
                  transform_scale_ue8m0)
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


_UE8M0_REQUANT = False


def set_ue8m0_requant(enabled: bool) -> None:
    """Stand-in for sglang's ``should_deepgemm_weight_requant_ue8m0`` (quantizer_fp8.py:103): the reference takes the
    power-of-two-scale branch of ``_quantize_param`` only when the rollout engine runs DeepGEMM with UE8M0 scales,
    which no engine on this hardware does - so it is off unless a caller switches it on here."""
    global _UE8M0_REQUANT
    _UE8M0_REQUANT = bool(enabled)


def ue8m0_requant_enabled() -> bool:
    return _UE8M0_REQUANT


def _quantize_param(name, weight, weight_block_size, transform_ue8m0=True):
    """-> [(name, qweight), (scale_name, scale)]; block scales are named ``.weight_scale_inv``, per-tensor
    scales ``.weight_scale`` (quantizer_fp8.py:98-118)."""
    assert name.endswith(".weight"), f"Expected weight parameter, got {name}"
    if weight_block_size is not None:
        if _UE8M0_REQUANT:
            qweight, scale = quant_weight_ue8m0(weight, weight_block_size=weight_block_size)
            if transform_ue8m0:
                scale = transform_scale_ue8m0(scale, mn=qweight.shape[-2])      # raises: NVIDIA-only layout
        else:
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
    if weight_block_size is not None and len(todo) > 1 and not _UE8M0_REQUANT and all(
            p.is_cuda and p.dim() == 2 and p.dtype == torch.bfloat16 and p.numel() for _, p in todo):
        outs = _group_cast([p for _, p in todo], weight_block_size)
        result = []
        for (n, _), (q, s) in zip(todo, outs):
            result += [(n, q), (n.replace(".weight", ".weight_scale_inv"), s)]
        return result

    result = []
    for n, p in todo:
        result.extend(_quantize_param(n, p, weight_block_size, transform_ue8m0))
    return result


class _QuantDesc(ctypes.Structure):
    """``wq_fp8_quant_desc``."""
    _fields_ = [("x", ctypes.c_void_p), ("y", ctypes.c_void_p), ("s", ctypes.c_void_p), ("M", ctypes.c_int64),
                ("N", ctypes.c_int64), ("sx_m", ctypes.c_int64), ("sx_n", ctypes.c_int64), ("sy_m", ctypes.c_int64)]


def _group_cast(weights, block_size):
    """``blockwise_cast_to_fp8_triton`` over the few tensors of one parameter with one launch -> [(qweight, scale)],
    fresh outputs (slices of one new allocation).  The descriptors travel in the kernel arguments
    (``wq_fp8_block_quant_few``): nothing is cached and nothing depends on where the inputs live, so a parameter
    that is gathered into fresh tensors on every sync costs the same as one that stays put."""
    bm, bn = int(block_size[0]), int(block_size[1])
    device = weights[0].device
    results = []
    lib = _lib.load()
    for g0 in range(0, len(weights), _lib.FP8_FEW_MAX):
        group = weights[g0:g0 + _lib.FP8_FEW_MAX]
        descs = (_QuantDesc * len(group))()
        layout, off = [], 0
        for d, w in zip(descs, group):
            M, N = w.shape
            tm, tn = ceildiv(M, bm), ceildiv(N, bn)
            q0 = off
            s0 = (q0 + M * N + 127) // 128 * 128          # codes of every tensor start on a 128-byte line
            off = (s0 + 4 * tm * tn + 127) // 128 * 128
            d.x, d.y, d.s, d.M, d.N, d.sx_m, d.sx_n, d.sy_m = w.data_ptr(), q0, s0, M, N, w.stride(0), w.stride(1), N
            layout.append((q0, M, N, s0, tm, tn))
        flat = torch.empty(off, dtype=torch.uint8, device=device)
        with torch.cuda.device(device):
            rc = lib.wq_fp8_block_quant_few(descs, len(group), flat.data_ptr(), bm, bn, _lib.FP8_MODE_TRITON,
                                            _lib.stream_ptr(device))
        _lib.check(rc, "quantize_params_fp8")
        results += [(flat[q0:q0 + M * N].view(FP8_DTYPE).view(M, N), flat[s0:s0 + 4 * tm * tn].view(torch.float32).view(tm, tn))
                    for q0, M, N, s0, tm, tn in layout]
    return results


# Work-item tables of quantize_grouped_weights, one per (expert count, shape, strides, block, device): address-free
# templates (see _tables.ResolvedTable), so the number of entries is the number of distinct grouped linears, not the
# number of allocations they have lived in.
_GROUP_TABLES: OrderedDict = OrderedDict()
_GROUP_LOCK = threading.Lock()
_GROUP_STATS = {"builds": 0, "hits": 0, "resolves": 0, "bytes": 0}
_GROUP_MAX_ENTRIES = 64
_GROUP_MAX_BYTES = 512 << 20


def plan_cache_info() -> dict:
    """Counters of the work-item table cache behind ``quantize_grouped_weights``: layouts built on the host, calls
    that found theirs, calls whose weights had moved (one address upload and one small launch each), device bytes held."""
    return dict(_GROUP_STATS, entries=len(_GROUP_TABLES))


def quantize_grouped_weights(weights, block_size=(128, 128), use_ue8m0: bool = False):
    """The expert weights of one grouped linear quantised by ONE launch straight into the stacked tensors a grouped GEMM
    reads: -> (qweight e4m3fn [E, N, K], scale float32 [E, ceil(N/bm), ceil(K/bn)]).

    Replaces the loop of ``_quantize_grouped_weights`` (slime/backends/megatron_utils/alignment/
    deepgemm_moe_forward.py:1383-1428), which calls ``ops.quantize_weight(weight, (128, 128))`` - that is
    ``blockwise_cast_to_fp8_triton``, or sglang's ``quant_weight_ue8m0`` with ``use_ue8m0`` - once per expert and copies
    every result into the stacked tensors: E launches, 2 E copies and a second pass over the quantised bytes.  Same
    bytes.  The per-tile table is cached per layout (expert count, shape, strides), not per address: weights that come
    back somewhere else cost one upload of E addresses and one small launch.  Calls must be ordered on one stream.
    All weights: 2-D bf16 on one GPU, one shape.  The reference's later ``requant_weight_ue8m0`` of the stacked
    tensors (sglang, Blackwell only) is not provided."""
    weights = list(weights)
    if not weights:
        raise ValueError("quantize_grouped_weights: no weights")
    bm, bn = int(block_size[0]), int(block_size[1])
    shape, device = tuple(weights[0].shape), weights[0].device
    for i, w in enumerate(weights):
        if w.dtype != torch.bfloat16:
            raise RuntimeError(f"weight{i} must be BF16, got {w.dtype}")
        if not w.is_cuda or w.device != device:
            raise RuntimeError(f"weight{i} must be on {device}, got {w.device}")
        if w.dim() != 2 or tuple(w.shape) != shape:
            raise RuntimeError(f"weight{i} has shape {tuple(w.shape)}, expected {shape}")
    E, (M, N) = len(weights), shape
    tm, tn = ceildiv(M, bm), ceildiv(N, bn)
    mode = _lib.FP8_MODE_UE8M0 if use_ue8m0 else _lib.FP8_MODE_TRITON
    if E * M * N == 0:
        return (torch.empty((E, M, N), dtype=FP8_DTYPE, device=device),
                torch.empty((E, tm, tn), dtype=torch.float32, device=device))
    key = ("stacked", bm, bn, device.index, shape, tuple(w.stride() for w in weights))
    ptrs = [w.data_ptr() for w in weights]
    s_base = (E * M * N + 15) // 16 * 16
    with _GROUP_LOCK:
        table = _GROUP_TABLES.get(key)
        if table is not None:
            _GROUP_TABLES.move_to_end(key)
            _GROUP_STATS["hits"] += 1
        else:
            rows = [[0, e * M * N, s_base + 4 * e * tm * tn, M, N, w.stride(0), w.stride(1), N] for e, w in enumerate(weights)]
            template, owner, _ = tile_table(rows, bm, bn)
            table = ResolvedTable(template, owner, E, device)
            _GROUP_TABLES[key] = table
            _GROUP_STATS["builds"] += 1
            _GROUP_STATS["bytes"] += table.device_bytes
            while (len(_GROUP_TABLES) > _GROUP_MAX_ENTRIES or _GROUP_STATS["bytes"] > _GROUP_MAX_BYTES) and len(_GROUP_TABLES) > 1:
                _, old = _GROUP_TABLES.popitem(last=False)
                _GROUP_STATS["bytes"] -= old.device_bytes
        if table.resolved_for != ptrs:
            table.resolve(np.asarray(ptrs, dtype=np.int64), tag=ptrs)
            _GROUP_STATS["resolves"] += 1
        flat = torch.empty(s_base + 4 * E * tm * tn, dtype=torch.uint8, device=device)
        with torch.cuda.device(device):
            rc = _lib.load().wq_fp8_bucket_convert(table.items.data_ptr(), table.n_items, flat.data_ptr(), bm, bn, mode,
                                                   _lib.stream_ptr(device))
    _lib.check(rc, "quantize_grouped_weights")
    return (flat[:E * M * N].view(FP8_DTYPE).view(E, M, N),
            flat[s_base:s_base + 4 * E * tm * tn].view(torch.float32).view(E, tm, tn))


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
           "set_ue8m0_requant", "ue8m0_requant_enabled", "plan_cache_info", "quantize_grouped_weights", "FP8_DTYPE"]
