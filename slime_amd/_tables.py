"""Work-item tables that outlive the addresses of their inputs.

The one-launch forms read one pre-resolved descriptor per work item.  Everything in such a table except the address of
the item's input follows from names, shapes and strides and is the same on every call, while the inputs of a weight
sync are fresh allocations each time once the model is sharded (gathered partitions and concatenated experts,
slime/backends/megatron_utils/update_weight/common.py:97,120).  A ``ResolvedTable`` keeps the table as a template whose
first word per item is a byte offset inside one of the inputs, plus the index of that input; ``resolve`` uploads the
inputs' current addresses (8 bytes each, through pinned staging) and lets ``wq_bucket_resolve_items`` add them on the
GPU.  A call whose inputs have not moved skips both.
"""

from __future__ import annotations

import numpy as np
import torch

from . import _lib

_STAGING_DEPTH = 4


class ResolvedTable:
    """``template``: int64 [n_items, width] (host), word 0 of a row = byte offset inside input ``owner[row]``;
    ``n_bases``: number of inputs.  ``items`` is the device table the launches read, valid for the addresses last
    passed to ``resolve``.  Calls must be ordered on one stream: ``items`` and the upload buffer are reused."""

    def __init__(self, template: torch.Tensor, owner: torch.Tensor, n_bases: int, device: torch.device):
        assert template.dim() == 2 and template.dtype == torch.int64 and owner.numel() == template.shape[0]
        self.device = device
        self.n_items, self.width = int(template.shape[0]), int(template.shape[1])
        self.template = template.contiguous().to(device)
        self.owner = owner.to(torch.int32).contiguous().to(device)
        self.items = torch.empty_like(self.template)
        self.bases = torch.empty(max(n_bases, 1), dtype=torch.int64, device=device)
        self._staging = [torch.empty(max(n_bases, 1), dtype=torch.int64).pin_memory() for _ in range(_STAGING_DEPTH)]
        self._events = [None] * _STAGING_DEPTH
        self._next = 0
        self.resolved_for = None            # whatever the caller passed as `tag` with the addresses now in `items`
        self.resolves = 0

    @property
    def device_bytes(self) -> int:
        return 2 * self.template.numel() * 8 + self.owner.numel() * 4 + self.bases.numel() * 8

    def resolve(self, bases: np.ndarray, tag=None) -> None:
        """``bases``: int64 addresses of the inputs, in the order ``owner`` indexes them."""
        k = self._next
        self._next = (k + 1) % _STAGING_DEPTH
        if self._events[k] is not None:
            self._events[k].synchronize()           # the upload that last used this staging buffer has finished
        host = self._staging[k]
        host.numpy()[:len(bases)] = bases
        stream = torch.cuda.current_stream(self.device)
        with torch.cuda.device(self.device):
            self.bases.copy_(host, non_blocking=True)
            ev = torch.cuda.Event()
            ev.record(stream)
            self._events[k] = ev
            rc = _lib.load().wq_bucket_resolve_items(self.template.data_ptr(), self.owner.data_ptr(), self.bases.data_ptr(),
                                                     self.n_items, self.width, self.items.data_ptr(), stream.cuda_stream)
        _lib.check(rc, "resolving a work-item table")
        self.resolved_for = tag
        self.resolves += 1
