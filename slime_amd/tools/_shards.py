"""Shard plumbing shared by the offline converters: reading safetensors shards, moving a shard's tensors to the
GPU and back, the index / config writers and the result collector."""

from __future__ import annotations

import json
import os
import shutil
import threading

import torch
from safetensors import safe_open
from safetensors.torch import save_file


def device() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("the converters run their arithmetic on the GPU; no GPU is visible and there is no CPU path")
    return torch.device("cuda", torch.cuda.current_device())


def read_shard(path: str) -> dict:
    """All tensors of one .safetensors file as CPU tensors (memory-mapped by safetensors)."""
    out = {}
    with safe_open(path, framework="pt", device="cpu") as f:
        for k in f.keys():
            out[k] = f.get_tensor(k)
    return out


def write_shard(tensors: dict, path: str, with_format_tag: bool = True) -> None:
    """The FP8 and INT4 converters tag their shards with metadata {"format": "pt"}
    (tools/convert_hf_to_fp8.py:161); the dequantising tool writes none (tools/fp8_cast_bf16.py:94)."""
    tensors = {k: v.contiguous() for k, v in tensors.items()}
    if with_format_tag:
        save_file(tensors, path, metadata={"format": "pt"})
    else:
        save_file(tensors, path)


def copy_side_files(input_path: str, output_path: str) -> None:
    """Everything in the checkpoint directory that is neither a shard nor a directory is copied verbatim
    (tools/convert_hf_to_fp8.py:170-172)."""
    for name in os.listdir(input_path):
        src = os.path.join(input_path, name)
        if not name.endswith(".safetensors") and not os.path.isdir(src):
            shutil.copyfile(src, os.path.join(output_path, name))


def list_shards(input_path: str) -> list:
    return sorted(f for f in os.listdir(input_path) if f.endswith(".safetensors"))


def locate_tensors(checkpoint_dir: str) -> dict:
    """{tensor name: shard file name} of a HF checkpoint directory.  ``model.safetensors.index.json`` decides when it
    exists; otherwise every shard's header is read (in sorted order, so a name stored twice resolves to the last
    shard).  FileNotFoundError when the directory holds neither."""
    index = os.path.join(checkpoint_dir, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index) as f:
            return dict(json.load(f)["weight_map"])
    shards = list_shards(checkpoint_dir)
    if not shards:
        raise FileNotFoundError(f"No safetensors checkpoint found in {checkpoint_dir}")
    where = {}
    for shard in shards:
        with safe_open(os.path.join(checkpoint_dir, shard), framework="pt", device="cpu") as f:
            for key in f.keys():
                where[key] = shard
    return where


class ConversionResult:
    """Thread-safe accumulator of the output index.  ``param_count`` reproduces the reference's quirk: it adds
    ``len(tensor)`` - the first dimension - of every output tensor (tools/convert_hf_to_fp8.py:110-114), and
    that number is what lands in ``metadata.total_size``."""

    def __init__(self):
        self.lock = threading.Lock()
        self.weight_map = {}
        self.param_count = 0
        self.modules_to_not_convert = []

    def add_result(self, filename: str, tensors: dict, module_names=()):
        with self.lock:
            for k, v in tensors.items():
                self.weight_map[k] = filename
                self.param_count += len(v)
            self.modules_to_not_convert.extend(module_names)


def write_index(output_path: str, result: ConversionResult) -> None:
    index = {"weight_map": result.weight_map, "metadata": {"total_size": result.param_count}}
    with open(os.path.join(output_path, "model.safetensors.index.json"), "w") as f:
        json.dump(index, f, indent=2)


def write_config(input_path: str, output_path: str, quantization_config: dict) -> None:
    src = os.path.join(input_path, "config.json")
    if os.path.exists(src):
        with open(src) as f:
            cfg = json.load(f)
        cfg["quantization_config"] = quantization_config
        with open(os.path.join(output_path, "config.json"), "w") as f:
            json.dump(cfg, f, indent=2)


def to_device(t: torch.Tensor, dev: torch.device) -> torch.Tensor:
    return t.to(dev, non_blocking=True)


class _HostStage(threading.local):
    """This thread's pinned staging memory for results on their way to a shard file.  A fresh pageable destination
    (``tensor.cpu()``) costs a page fault per 4 KiB and a bounce copy: 4 GB/s on a machine whose link does 55 GB/s into
    pinned memory.  The memory is a bump allocator over grow-only chunks; ``reset`` (start of the next shard on this
    thread) rewinds it and folds the chunks into one, so from the second shard on a worker allocates nothing."""

    chunk_bytes = 256 << 20

    def __init__(self):
        self.chunks, self.used, self.cur = [], 0, 0

    def reset(self):
        total = sum(c.numel() for c in self.chunks)
        if len(self.chunks) > 1:
            self.chunks = []                  # release before asking for the sum of them in one piece
            self.chunks = [self._alloc(total)]
        self.used = self.cur = 0

    @staticmethod
    def _alloc(nbytes: int) -> torch.Tensor:
        try:
            return torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
        except RuntimeError:                  # the host refuses to lock more memory: pageable staging still works
            return torch.empty(nbytes, dtype=torch.uint8)

    def take(self, nbytes: int) -> torch.Tensor:
        nbytes_al = -(-max(nbytes, 1) // 256) * 256
        while self.cur < len(self.chunks) and self.used + nbytes_al > self.chunks[self.cur].numel():
            self.cur, self.used = self.cur + 1, 0
        if self.cur == len(self.chunks):
            self.chunks.append(self._alloc(max(nbytes_al, self.chunk_bytes)))
            self.used = 0
        piece = self.chunks[self.cur][self.used:self.used + nbytes]
        self.used += nbytes_al
        return piece


_stage = _HostStage()


def begin_shard() -> None:
    """Call at the start of every shard: host tensors handed out by ``to_host`` for the previous shard of this thread
    are dead from here on (their memory is reused)."""
    _stage.reset()


def to_host(*tensors: torch.Tensor):
    """Device tensors -> host tensors of the same shape and dtype inside this thread's pinned staging memory; one
    synchronisation for all of them.  Valid until this thread's next ``begin_shard``."""
    out = []
    for t in tensors:
        t = t.contiguous()
        h = _stage.take(t.numel() * t.element_size()).view(t.dtype).view(t.shape)
        h.copy_(t, non_blocking=True)
        out.append(h)
    if tensors:
        torch.cuda.current_stream(tensors[0].device).synchronize()
    return out[0] if len(out) == 1 else tuple(out)


def copy_matching_files(input_path: str, output_path: str, keep, skip=()) -> None:
    """Copies (with metadata) the plain files of a checkpoint directory for which ``keep(name)`` holds."""
    for name in os.listdir(input_path):
        src = os.path.join(input_path, name)
        if name not in skip and os.path.isfile(src) and keep(name):
            shutil.copy2(src, os.path.join(output_path, name))


def write_index_of_directory(output_path: str) -> None:
    """model.safetensors.index.json rebuilt from the shards that are in the directory, with empty metadata."""
    weight_map = {}
    for fname in list_shards(output_path):
        with safe_open(os.path.join(output_path, fname), framework="pt") as reader:
            for key in reader.keys():
                weight_map[key] = fname
    with open(os.path.join(output_path, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f, indent=2)
