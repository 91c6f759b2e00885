"""HF safetensors checkpoint reader that dequantises block-scaled FP8 weights on read, on the GPU.

Same interface as the reference's ``SafetensorReader`` (slime/backends/megatron_utils/hf_to_megatron/common.py:13-56):
the HF -> Megatron loaders ask for one tensor at a time by HF name, ``name in reader`` tells whether the checkpoint
has it, and only the most recently returned tensor is cached.  A float8_e4m3fn tensor that has a
``<name>_scale_inv`` sibling comes back as bf16 ``weight * bf16(scale)[block]``.  The reference computes that on the host
with a pad / view / in-place multiply (four full-size temporaries); here codes and scales are uploaded and one HIP
kernel writes the bf16 result (``weight_dequant_bf16_scale``: e4m3 -> bf16 exactly, scale rounded to bf16, product
rounded once - the same bits).  Everything else is returned as stored.
"""

from __future__ import annotations

import os

import torch
from safetensors import safe_open

from .fp8 import FP8_DTYPE, weight_dequant_bf16_scale
from .tools._shards import locate_tensors


class SafetensorReader:
    """``SafetensorReader(path).get_tensor(name)``.

    Every tensor comes back on the host, as from the reference's reader, so a loader may concatenate dequantised and
    unquantised tensors of a partly converted checkpoint.  ``device="cuda"`` leaves dequantised weights on the GPU
    instead (one PCIe crossing less when the caller copies them into GPU parameters anyway); tensors that need no
    dequantisation are host tensors either way."""

    def __init__(self, path, device=None):
        self.path = os.fspath(path)
        self.weight_map = locate_tensors(self.path)
        self._handles = {}                 # shard file name -> open safetensors handle
        self._keep_on_gpu = device is not None and torch.device(device).type == "cuda"
        self._last = (None, None)          # name and tensor of the most recent request

    def __contains__(self, name: str) -> bool:
        return name in self.weight_map

    def _stored(self, name: str) -> torch.Tensor:
        shard = self.weight_map.get(name)
        if shard is None:
            raise KeyError(f"HuggingFace checkpoint does not contain {name!r}")
        handle = self._handles.get(shard)
        if handle is None:
            handle = self._handles[shard] = safe_open(os.path.join(self.path, shard), framework="pt", device="cpu")
        return handle.get_tensor(name)

    def get_tensor(self, name: str) -> torch.Tensor:
        if self._last[0] == name:
            return self._last[1]
        tensor = self._stored(name)
        if tensor.element_size() == 1 and f"{name}_scale_inv" in self.weight_map:
            tensor = self._dequantised(name, tensor)
        self._last = (name, tensor)
        return tensor

    def _dequantised(self, name: str, codes: torch.Tensor) -> torch.Tensor:
        # The reference converts the stored tensor numerically (``.to(bfloat16)``), which for float8_e4m3fn is the
        # decoding the kernel performs.  Other one-byte dtypes (int8, uint8, float8_e5m2) would convert to other values
        # than their bytes read as e4m3fn, so they are refused rather than reinterpreted.
        if codes.dtype != FP8_DTYPE:
            raise TypeError(f"{name}: a block-scaled tensor must be stored as float8_e4m3fn to be dequantised here, "
                            f"got {codes.dtype}")
        if not torch.cuda.is_available():
            raise RuntimeError("SafetensorReader dequantises on the GPU; no GPU is visible and there is no CPU path")
        gpu = torch.device("cuda", torch.cuda.current_device())
        scale = self._stored(f"{name}_scale_inv").to(torch.float32).contiguous()
        out = weight_dequant_bf16_scale(codes.contiguous().to(gpu, non_blocking=True), scale.to(gpu, non_blocking=True))
        return out if self._keep_on_gpu else out.cpu()
