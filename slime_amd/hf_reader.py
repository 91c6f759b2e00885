"""HF safetensors checkpoint reader that dequantises block-scaled FP8 weights on read, on the GPU.

Mirror of ``SafetensorReader`` (slime/backends/megatron_utils/hf_to_megatron/common.py:13-56): the HF -> Megatron
loaders ask it for one tensor at a time by HF name; a one-byte tensor that has a ``<name>_scale_inv`` sibling is
returned as bf16 ``weight * bf16(scale)[block]``.  The reference does that with a pad / view / in-place multiply on the
host (four full-size temporaries); here the codes and the scales are uploaded and one HIP kernel writes the bf16
result (``weight_dequant_bf16_scale``: e4m3 -> bf16 exactly, scale rounded to bf16, product rounded once - the same
bits).  Everything else is returned as stored.  The last tensor is cached, as in the reference.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors import safe_open

from .fp8 import weight_dequant_bf16_scale


class SafetensorReader:
    """``SafetensorReader(path).get_tensor(name)``.  ``device``: where dequantised weights are left - the current GPU
    by default (the loader copies them into GPU parameters anyway), or ``"cpu"`` to hand back a host tensor like the
    reference does.  Tensors that need no dequantisation come back as the file holds them (host tensors)."""

    def __init__(self, path, device=None):
        self.path = Path(path)
        index_path = self.path / "model.safetensors.index.json"
        if index_path.is_file():
            with index_path.open() as index_file:
                self.weight_map = json.load(index_file)["weight_map"]
        else:
            files = sorted(self.path.glob("*.safetensors"))
            if not files:
                raise FileNotFoundError(f"No safetensors checkpoint found in {self.path}")
            self.weight_map = {}
            for file in files:
                with safe_open(file, framework="pt", device="cpu") as tensors:
                    self.weight_map.update(dict.fromkeys(tensors.keys(), file.name))
        self._files = {}
        self._device = device
        self._last = None              # (name, tensor): only the most recent tensor is kept, as with the reference's lru_cache(1)

    def __contains__(self, name: str) -> bool:
        return name in self.weight_map

    def _open(self, filename: str):
        if filename not in self._files:
            self._files[filename] = safe_open(self.path / filename, framework="pt", device="cpu")
        return self._files[filename]

    def get_tensor(self, name: str) -> torch.Tensor:
        if self._last is not None and self._last[0] == name:
            return self._last[1]
        try:
            filename = self.weight_map[name]
        except KeyError as exc:
            raise KeyError(f"HuggingFace checkpoint does not contain {name!r}") from exc
        tensor = self._open(filename).get_tensor(name)
        scale_name = f"{name}_scale_inv"
        if tensor.element_size() == 1 and scale_name in self:
            if not torch.cuda.is_available():
                raise RuntimeError("SafetensorReader dequantises on the GPU; no GPU is visible and there is no CPU path")
            gpu = torch.device("cuda", torch.cuda.current_device())
            scale = self._open(self.weight_map[scale_name]).get_tensor(scale_name)
            codes = tensor.view(torch.float8_e4m3fn).contiguous().to(gpu, non_blocking=True)
            tensor = weight_dequant_bf16_scale(codes, scale.to(torch.float32).contiguous().to(gpu, non_blocking=True))
            if self._device is not None and torch.device(self._device).type == "cpu":
                tensor = tensor.cpu()
        self._last = (name, tensor)
        return tensor
