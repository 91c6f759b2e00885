"""The one digest of the delta publisher that stays a host computation: blake3, a tree hash with its own package
(slime/utils/disk_delta.py:46-49 imports ``blake3`` the same way).  adler32 and xxh3-128 are computed on the GPU
(``slime_amd.delta.checksum``)."""

from __future__ import annotations

import torch


def host_checksum(algorithm: str, buf: torch.Tensor) -> str:
    if algorithm != "blake3":
        raise KeyError(f"unknown checksum algorithm {algorithm!r}")
    import blake3

    h = blake3.blake3()
    h.update(buf.detach().contiguous().view(torch.uint8).reshape(-1).cpu().numpy())
    return h.hexdigest()
