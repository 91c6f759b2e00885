"""Host-resident weights through the GPU quantisers: double-buffered pinned H2D -> kernel -> D2H.

The offline converters of the reference load a whole safetensors shard onto the device, quantise it tensor by
tensor and write it back (tools/convert_hf_to_fp8.py:118-163, tools/convert_hf_to_int4_direct.py:169-206,
tools/fp8_cast_bf16.py:68-100).  With host-resident data the path is PCIe-bound, so the only thing that matters is
that uploads, kernels and downloads overlap.  ``BucketPipeline`` does that for a stream of equally-shaped or
ragged buckets:

* ``depth`` pinned host staging buffers and ``depth`` device buffers per direction (allocated once);
* an upload stream, the caller's compute stream and a download stream, all at default priority, ordered with events;
* the kernels are the same grouped launches the resident path uses (``Fp8QuantPlan`` etc. are not needed here
  because each bucket is one 2-D tensor).

Pinned memory is allocated (``pin_memory=True``), never registered after the fact.
"""

from __future__ import annotations

from typing import Callable, Iterable, Iterator

import torch


class BucketPipeline:
    """Runs ``kernel(dev_in_bucket) -> tuple of device tensors`` over host buckets with overlap.

    ``process(buckets)`` takes an iterable of CPU tensors (any dtype, contiguous) and yields, in order, tuples of
    CPU tensors holding the kernel's outputs.  Input buckets must not exceed ``max_in_bytes``; each output must
    not exceed ``max_out_bytes``.

    Buffer lifetimes.  The yielded tensors are views of pinned staging buffers, of which there are ``depth + 1``
    sets: a result stays intact while the iterator is advanced ONCE more (so the previous result may be held while
    the current one is worked on) and is overwritten, asynchronously, from the second advance on - copy what has to
    live longer.  Input staging: ``staging_buffer(slot)`` of bucket ``i`` is ``slot = i % depth``; ``process`` pulls
    bucket ``i`` from the iterable only after bucket ``i - depth`` (the previous user of that slot) has completely
    left the GPU, so a generator may refill the buffer right before yielding it.
    """

    def __init__(self, device: torch.device, kernel: Callable[[torch.Tensor], tuple], max_in_bytes: int,
                 max_out_bytes: int, n_outputs: int, depth: int = 2, download: bool = True):
        if device.type != "cuda":
            raise RuntimeError("BucketPipeline needs a GPU device; there is no CPU path")
        self.device, self.kernel, self.depth, self.download, self.n_outputs = device, kernel, depth, download, n_outputs
        self.max_in_bytes, self.max_out_bytes = int(max_in_bytes), int(max_out_bytes)
        self.h_in = [torch.empty(self.max_in_bytes, dtype=torch.uint8, pin_memory=True) for _ in range(depth)]
        self.d_in = [torch.empty(self.max_in_bytes, dtype=torch.uint8, device=device) for _ in range(depth)]
        # one more set of output buffers than buckets in flight: the set of the result handed out last is not the
        # one the next bucket downloads into
        self.h_out = [[torch.empty(self.max_out_bytes, dtype=torch.uint8, pin_memory=True) for _ in range(n_outputs)]
                      for _ in range(depth + 1)] if download else None
        self.up = torch.cuda.Stream(device)
        self.down = torch.cuda.Stream(device)
        self.ev_uploaded = [torch.cuda.Event() for _ in range(depth)]
        self.ev_computed = [torch.cuda.Event() for _ in range(depth)]
        self.ev_downloaded = [torch.cuda.Event() for _ in range(depth + 1)]
        self.kernel_events = []   # (start, end) pairs when time_kernels is set
        self.time_kernels = False

    def _stage(self, slot: int, bucket: torch.Tensor) -> torch.Tensor:
        nbytes = bucket.numel() * bucket.element_size()
        if nbytes > self.max_in_bytes:
            raise ValueError(f"bucket of {nbytes} bytes exceeds the pipeline's {self.max_in_bytes}")
        if bucket.device.type != "cpu" or not bucket.is_contiguous():
            raise ValueError("buckets must be contiguous CPU tensors")
        flat = bucket.view(-1).view(torch.uint8)
        # host copy into pinned staging (skipped when the caller already hands us our own staging buffer)
        if flat.data_ptr() != self.h_in[slot].data_ptr():
            self.h_in[slot][:nbytes].copy_(flat)
        return self.h_in[slot][:nbytes]

    def staging_buffer(self, slot: int) -> torch.Tensor:
        """Pinned input buffer of ``slot`` (0..depth-1): fill it directly to avoid the extra host copy."""
        return self.h_in[slot]

    def process(self, buckets: Iterable[torch.Tensor]) -> Iterator[tuple]:
        compute = torch.cuda.current_stream(self.device)
        pending = []  # (input slot, output slot, outputs on device, their pinned host views)
        it = iter(buckets)
        i = 0
        while True:
            slot = i % self.depth
            if i >= self.depth:
                # the slot is reused: its previous bucket must have left the GPU (uploaded, computed, downloaded) before
                # the iterable is asked for the next bucket - it may refill this slot's staging buffer
                yield self._finish(pending.pop(0))
            try:
                bucket = next(it)
            except StopIteration:
                break
            staged = self._stage(slot, bucket)
            if i >= self.depth:
                # d_in[slot] may be overwritten only after the kernel of its previous bucket has read it
                self.up.wait_event(self.ev_computed[slot])
            with torch.cuda.stream(self.up):
                d_in = self.d_in[slot][:staged.numel()]
                d_in.copy_(staged, non_blocking=True)
                self.ev_uploaded[slot].record(self.up)
            compute.wait_event(self.ev_uploaded[slot])
            dev_bucket = d_in.view(bucket.dtype).view(bucket.shape)
            if self.time_kernels:
                s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                s.record(compute)
            outs = self.kernel(dev_bucket)
            if self.time_kernels:
                e.record(compute)
                self.kernel_events.append((s, e))
            self.ev_computed[slot].record(compute)
            host_outs = None
            if self.download:
                self.down.wait_event(self.ev_computed[slot])
                oslot = i % (self.depth + 1)
                host_outs = []
                with torch.cuda.stream(self.down):
                    for k, o in enumerate(outs):
                        nbytes = o.numel() * o.element_size()
                        if nbytes > self.max_out_bytes:
                            raise ValueError(f"output of {nbytes} bytes exceeds the pipeline's {self.max_out_bytes}")
                        h = self.h_out[oslot][k][:nbytes]
                        h.copy_(o.contiguous().view(-1).view(torch.uint8), non_blocking=True)
                        o.record_stream(self.down)
                        host_outs.append(h.view(o.dtype).view(o.shape))
                    self.ev_downloaded[oslot].record(self.down)
            pending.append((slot, oslot if self.download else None, outs, host_outs))
            i += 1
        while pending:
            yield self._finish(pending.pop(0))

    def _finish(self, item):
        slot, oslot, outs, host_outs = item
        if self.download:
            self.ev_downloaded[oslot].synchronize()
            return tuple(host_outs)
        self.ev_computed[slot].synchronize()
        return tuple(outs)

    def kernel_ms(self) -> float:
        """Sum of kernel times of the buckets processed with ``time_kernels`` set (call after a synchronize)."""
        return sum(s.elapsed_time(e) for s, e in self.kernel_events)


def fp8_block_quant_kernel(block_size=(128, 128), mode: int | None = None) -> Callable[[torch.Tensor], tuple]:
    """Kernel adaptor for BucketPipeline: bf16 [M,N] -> (e4m3fn [M,N], fp32 scale_inv)."""
    from . import arith
    from .fp8 import _block_quant

    def run(w: torch.Tensor):
        m = arith.fp8_torch_mode() if mode is None else mode
        return _block_quant(w, int(block_size[0]), int(block_size[1]), m, "stream.fp8_block_quant")

    return run


def int4_pack_kernel(group_size: int = 128) -> Callable[[torch.Tensor], tuple]:
    """Kernel adaptor for BucketPipeline: bf16 [M,N] -> (packed int32 [M,N/8], bf16 scale [M,N/group])."""
    from .int4 import pack_layer

    def run(w: torch.Tensor):
        packed, scale, _ = pack_layer(w, group_size, True)
        return packed, scale

    return run
