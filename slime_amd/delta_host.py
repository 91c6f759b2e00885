"""Host-side digests for the delta publisher: the sequential hash functions the GPU does not compute
(slime/utils/disk_delta.py:40-58: xxh3-128 via ``xxhash``, blake3 via ``blake3``)."""

from __future__ import annotations

import torch


def host_checksum(algorithm: str, buf: torch.Tensor) -> str:
    data = buf.detach().contiguous().view(torch.uint8).reshape(-1).cpu().numpy()
    if algorithm == "xxh3-128":
        import xxhash

        h = xxhash.xxh3_128()
    elif algorithm == "blake3":
        import blake3

        h = blake3.blake3()
    else:
        raise KeyError(f"unknown checksum algorithm {algorithm!r}")
    h.update(data)
    return h.hexdigest()
