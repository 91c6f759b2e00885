"""A whole weight-sync bucket converted, quantised and flattened by ONE kernel launch.

The reference's hot loop is one ``convert_to_hf`` / ``quantize_params`` call per Megatron parameter
(``HfWeightIteratorDirect._convert_to_hf_named_tensors``, slime/backends/megatron_utils/update_weight/
hf_weight_iterator_direct.py:50-67) - a kernel launch or a dozen per tensor - followed by a second pass that copies
every result into one uint8 buffer (``FlattenedTensorBucket(named_tensors=...)`` in ``_build_flattened_tensor_data``,
update_weight_from_tensor.py:30-48).  ``BucketConverter.convert`` takes the bucket after name conversion - a list of
``(megatron_name, [(hf_name, tensor), ...])`` - applies the routing of ``quantize_params`` (processors/__init__.py:6-22,
quantizer_fp8.py:10-95, quantizer_compressed_tensors.py:268-297) and issues one launch whose work items either quantise
a tile / a run of groups straight into its place in the flat buffer or copy a piece of a pass-through tensor there.  The
result has the layout the bucket consumer reads: one uint8 tensor plus ``(name, shape, dtype, start_idx, end_idx, numel)``
per tensor, names in the order the per-parameter loop produces them, tensors packed back to back.

The per-item table is built once per bucket *layout* (names, shapes, strides and dtypes) as a template that holds no
address: inputs appear in it as (tensor index, byte offset).  On every sync the addresses of the bucket's tensors are
compared with the ones the resolved table was made for; when any moved - which is every sync once the model is sharded,
because gathered parameters are fresh allocations (update_weight/common.py:97,120) - the addresses are uploaded (8 bytes
per tensor) and one small launch adds them to the template (``wq_bucket_resolve_items``).  Destinations in the table are
offsets, so every call can write into a fresh buffer (the reference warns against reusing the IPC-facing one,
update_weight_from_tensor.py:39-43) or into ``out=``.

Tensors are packed back to back exactly as ``FlattenedTensorBucket`` packs them.  A bucket in which that puts a tensor at
an offset that is not a multiple of its element size (an odd number of one-byte elements ahead of a wider tensor) is
converted by the per-parameter loop and concatenated with ``torch.cat``, as the reference does.
"""

from __future__ import annotations

import json
from collections import OrderedDict
from typing import NamedTuple, Sequence

import numpy as np
import torch

from . import _lib
from ._tables import ResolvedTable
from .fp8 import FP8_DTYPE, ceildiv, tile_table
from .int4 import item_table, zero_point_rows
from .processors import _fp8_route, _is_ignored, quantize_params, ue8m0_requant_enabled

_COPY = _lib.BUCKET_COPY_BYTES
_ELEMENT_SIZE: dict = {}


class FlattenedTensorMetadata(NamedTuple):
    """One entry of ``FlattenedTensorBucket.get_metadata()``: the tensor is
    ``flattened_tensor[start_idx:end_idx].view(dtype).reshape(shape)``; ``numel`` counts bytes.  (An immutable record
    with the fields of sglang's dataclass; a named tuple because a bucket builds tens of thousands of them.)"""
    name: str
    shape: torch.Size
    dtype: torch.dtype
    start_idx: int
    end_idx: int
    numel: int


class FlattenedBucket:
    """The pair the bucket consumer receives (``{"flattened_tensor": ..., "metadata": ...}``,
    update_weight_from_tensor.py:44-48), with ``FlattenedTensorBucket``'s accessors."""

    supports_multi_dtypes = True

    def __init__(self, flattened_tensor: torch.Tensor, metadata: Sequence[FlattenedTensorMetadata], launches: int = 0):
        self.flattened_tensor = flattened_tensor
        self.metadata = metadata if isinstance(metadata, list) else list(metadata)     # shared with the cached plan: read-only
        self.launches = launches            # kernel launches this bucket cost (diagnostic)

    def get_flattened_tensor(self) -> torch.Tensor:
        return self.flattened_tensor

    def get_metadata(self):
        return self.metadata

    def reconstruct_tensors(self):
        """-> [(name, tensor)]: views into the flat buffer, in bucket order."""
        return [(m.name, self.flattened_tensor[m.start_idx:m.end_idx].view(m.dtype).reshape(m.shape))
                for m in self.metadata]


def flatten_named_tensors(named_tensors) -> FlattenedBucket:
    """What ``FlattenedTensorBucket(named_tensors=...)`` builds - every tensor flattened to bytes, concatenated in order -
    with torch ops.  Used for buckets the one-launch path does not cover, and by the tests as the expected layout."""
    if not named_tensors:
        return FlattenedBucket(torch.empty(0, dtype=torch.uint8, device=torch.device("cuda", torch.cuda.current_device())), [])
    meta, parts, off = [], [], 0
    for name, t in named_tensors:
        b = t.detach().contiguous().flatten().view(torch.uint8)
        meta.append(FlattenedTensorMetadata(name, t.shape, t.dtype, off, off + b.numel(), b.numel()))
        parts.append(b)
        off += b.numel()
    return FlattenedBucket(torch.cat(parts, dim=0), meta, launches=len(parts) + 1)


class _Layout:
    """Everything about a bucket that does not depend on where its inputs live this sync."""
    __slots__ = ("kind", "block", "group", "device", "metadata", "total_bytes", "n_tensors", "n_items", "table",
                 "table_off_lines", "slot_src", "align", "const_base", "keepalive", "late_copies", "zero_bytes", "zp_rows", "zp_start",
                 "zp_words", "n_zp", "fallback")


class BucketConverter:
    """Converts buckets of one model under one ``quantization_config``; see the module docstring.

    ``convert(params)`` -> ``FlattenedBucket``.  ``params`` is a list ``[(megatron_name, [(hf_name, tensor), ...]), ...]`` -
    what ``_convert_to_hf_core`` yields per Megatron parameter.  Tensors the one-launch kernels do not take
    (FP8: not 2-D bf16 on the GPU; INT4: not contiguous 16-byte aligned bf16 with 32 / 64 / 128 groups; per-tensor FP8
    configurations) go through the per-tensor functions first and are copied in by the same launch, so
    the result is always what the per-parameter loop gives.

    Calls of one converter must be ordered on one stream (or by the caller): the resolved work-item table and the
    address upload buffer of a layout are reused from call to call.
    """

    def __init__(self, args=None, quantization_config=None, transform_ue8m0: bool = True, max_cached_plans: int = 256):
        self.args = args
        self.config = quantization_config
        self.transform_ue8m0 = transform_ue8m0
        self._config_key = json.dumps(quantization_config, sort_keys=True, default=str)
        self._layouts: OrderedDict = OrderedDict()
        self._max = int(max_cached_plans)
        self.plan_builds = 0            # layouts built on the host (names, shapes, offsets, the per-item template)
        self.resolves = 0               # syncs whose inputs had moved: one address upload + one resolve launch each
        self.time_kernels = False       # when set, convert() brackets its launch with events (kernel_ms())
        self.kernel_events = []
        method = None if quantization_config is None else quantization_config["quant_method"]
        self._method = method if method in ("fp8", "compressed-tensors") else None
        if self._method == "fp8":
            assert quantization_config.get("fmt", "e4m3") == "e4m3", f"Unsupported FP8 format: {quantization_config.get('fmt')}"
            assert quantization_config["activation_scheme"] == "dynamic"
            self._block = quantization_config.get("weight_block_size", None)
        elif self._method == "compressed-tensors":
            w_cfg = quantization_config["config_groups"]["group_0"]["weights"]
            self._group, self._sym = w_cfg["group_size"], w_cfg["symmetric"]
            self._ignore = quantization_config.get("ignore", [])

    # ------------------------------------------------------------------ routing (what the per-parameter loop decides)

    def _route(self, megatron_name, converted):
        """-> list of ("quant" | "pass" | "loop", hf_name, tensor, index in `converted`).  "loop": quantised, but by the
        per-tensor function."""
        if self._method == "fp8":
            route = _fp8_route(megatron_name)
            if route is None:
                return [("pass", n, t, ci) for ci, (n, t) in enumerate(converted)]
            ops = []
            for ci, (n, t) in enumerate(converted):
                if route == "skip_scales" and n.endswith("_scale"):
                    continue
                assert n.endswith(".weight"), f"Expected weight parameter, got {n}"
                one_launch = (self._block is not None and not ue8m0_requant_enabled() and t.is_cuda
                              and t.dim() == 2 and t.dtype == torch.bfloat16 and t.numel() > 0)
                ops.append(("quant" if one_launch else "loop", n, t, ci))
            return ops
        if self._method == "compressed-tensors":
            ops = []
            for ci, (n, t) in enumerate(converted):
                if _is_ignored(n, self._ignore) or not n.endswith(".weight") or t.dim() < 2:
                    ops.append(("pass", n, t, ci))
                    continue
                one_launch = (t.is_cuda and t.dim() == 2 and t.dtype == torch.bfloat16 and t.is_contiguous()
                              and t.data_ptr() % 16 == 0 and self._group in (32, 64, 128) and t.numel() > 0
                              and t.shape[1] % self._group == 0 and (self._sym or t.shape[0] % 8 == 0))
                ops.append(("quant" if one_launch else "loop", n, t, ci))
            return ops
        return [("pass", n, t, ci) for ci, (n, t) in enumerate(converted)]

    # ------------------------------------------------------------------ layout

    @staticmethod
    def _key(params):
        """Identity of a bucket's layout: everything but the addresses - names, shapes, dtypes, devices and strides.
        Built from flat passes over the tensors (a few hundred nanoseconds each); ``Tensor.stride()`` is by far the
        slowest of these accessors, so it is read for non-contiguous tensors only."""
        flat = [t for _, conv in params for _, t in conv]
        contiguous = [t.is_contiguous() for t in flat]
        return (tuple([mn for mn, _ in params]), tuple([len(conv) for _, conv in params]),
                tuple([n for _, conv in params for n, _ in conv]), tuple([t.shape for t in flat]),
                tuple([t.dtype for t in flat]), tuple([t.device for t in flat]), tuple(contiguous),
                tuple([t.stride() for t, c in zip(flat, contiguous) if not c]))

    def _build(self, params) -> _Layout:
        self.plan_builds += 1
        device = None
        for _, conv in params:
            for _, t in conv:
                if t.is_cuda:
                    device = t.device
                    break
            if device is not None:
                break
        if device is None:
            raise RuntimeError("BucketConverter: the bucket holds no GPU tensor; there is no CPU path")
        fp8 = self._method != "compressed-tensors"          # pass-through-only buckets use the FP8 launch's copy items
        plan = _Layout()
        asym = not fp8 and not self._sym
        plan.kind = "fp8" if fp8 else ("int4_asym" if asym else "int4")
        plan.block = tuple(int(b) for b in self._block) if (self._method == "fp8" and self._block is not None) else (128, 128)
        plan.group = int(self._group) if self._method == "compressed-tensors" else 128
        plan.fallback = False
        bm, bn = plan.block

        flat_index, k = {}, 0                           # (parameter, converted tensor) -> position among all tensors
        for pi, (_, conv) in enumerate(params):
            for ci in range(len(conv)):
                flat_index[(pi, ci)] = k
                k += 1
        plan.n_tensors = k
        slot_src, align = [], []                        # per input the launch reads: its position, its alignment mask

        def slot(pi, ci, mask):
            slot_src.append(flat_index[(pi, ci)])
            align.append(mask)
            return len(slot_src) - 1

        meta, off = [], 0
        quant_rows, copy_rows, late = [], [], []       # table rows per tensor; late = results only known at run time
        shape_rows, zp_entries, zero_off = [], [], 0

        def place(name, shape, dtype):
            """The next tensor of the flat buffer, back to back as FlattenedTensorBucket packs them."""
            nonlocal off
            esz = _ELEMENT_SIZE.get(dtype) or _ELEMENT_SIZE.setdefault(dtype, torch.empty((), dtype=dtype).element_size())
            if off % esz:
                # an odd-sized tensor ahead of a wider one: neither the kernels nor a consumer's .view(dtype) can
                # address the wider tensor at this offset, and padding would not be the reference's layout
                plan.fallback = True
            nbytes = esz
            for d in shape:
                nbytes *= int(d)
            meta.append(FlattenedTensorMetadata(name, shape if type(shape) is torch.Size else torch.Size(shape), dtype, off, off + nbytes, nbytes))
            start = off
            off += nbytes
            return start, nbytes

        def add_copy(name, t, pi, ci):
            start, nbytes = place(name, t.shape, t.dtype)
            if not nbytes:
                return
            if t.is_cuda and t.device == device and t.is_contiguous():
                copy_rows.append((len(meta) - 1, slot(pi, ci, 0), start, nbytes))
            else:
                late.append((len(meta) - 1, pi, ci, None))

        for pi, (mn, conv) in enumerate(params):
            for op, n, t, ci in self._route(mn, conv):
                if op == "pass":
                    add_copy(n, t, pi, ci)
                elif op == "loop":
                    # per-tensor function at run time (here only for the shapes of its outputs); copied into place afterwards
                    outs = quantize_params(self.args, mn, [(n, t)], self.config, self.transform_ue8m0)
                    for on, ot in outs:
                        place(on, ot.shape, ot.dtype)
                        late.append((len(meta) - 1, pi, ci, on))
                elif fp8:
                    M, N = t.shape
                    y0, _ = place(n, (M, N), FP8_DTYPE)
                    s0, _ = place(n.replace(".weight", ".weight_scale_inv"), (ceildiv(M, bm), ceildiv(N, bn)), torch.float32)
                    quant_rows.append((len(meta) - 2, slot(pi, ci, 0), [0, y0, s0, M, N, t.stride(0), t.stride(1), N]))
                else:
                    M, N = t.shape
                    if asym:        # zero points first, as the per-parameter loop emits them
                        G = N // plan.group
                        z0, _ = place(n.replace(".weight", ".weight_zero_point"), (G, M // 8), torch.int32)
                        zp_entries.append((zero_off, z0, M, G))
                    p0, _ = place(n.replace(".weight", ".weight_packed"), (M, N // 8), torch.int32)
                    s0, _ = place(n.replace(".weight", ".weight_scale"), (M, N // plan.group), torch.bfloat16)
                    h0, _ = place(n.replace(".weight", ".weight_shape"), (2,), torch.int32)
                    if asym:
                        quant_rows.append((len(meta) - 4, slot(pi, ci, 15), [0, p0, s0, zero_off, M * N // plan.group]))
                        zero_off += (2 * M * G + 15) // 16 * 16
                    else:
                        quant_rows.append((len(meta) - 3, slot(pi, ci, 15), [0, p0, s0, M * N // plan.group]))
                    shape_rows.append((len(meta) - 1, h0, (M, N)))

        plan.total_bytes = off
        plan.metadata = meta
        plan.late_copies = late
        plan.device = device
        plan.keepalive = []
        plan.n_items, plan.table, plan.table_off_lines = 0, None, None
        plan.zero_bytes, plan.n_zp = zero_off, len(zp_entries)
        if plan.fallback:
            return plan

        const_slot = len(slot_src)                      # one more base: the table of weight_shape values the layout owns
        plan.const_base = 0
        if shape_rows:
            shapes = torch.tensor([sh for _, _, sh in shape_rows], dtype=torch.int32).to(device)
            plan.keepalive.append(shapes)
            plan.const_base = shapes.data_ptr()
            for k, (mi, h0, _) in enumerate(shape_rows):
                copy_rows.append((mi, const_slot, h0, 8, 8 * k))

        # ---- one template row per work item, in bucket order (ordered by the metadata index of the item's first
        # output); word 0 is the item's byte offset inside its input tensor, `owner` says which tensor that is
        width = 8 if fp8 else (5 if asym else 4)
        blocks, order, owners = [], [], []
        if quant_rows:
            first = torch.tensor([mi for mi, _, _ in quant_rows], dtype=torch.int64)
            row_slot = torch.tensor([s for _, s, _ in quant_rows], dtype=torch.int64)
            rows = [r for _, _, r in quant_rows]
            if asym:
                # x, packed, scale and the zero scratch advance with the item; n_groups is what is left of the tensor
                full = torch.tensor(rows, dtype=torch.int64)
                table4, owner, local = item_table(full[:, [0, 1, 2, 4]], plan.group)
                zcol = full[owner, 3] + local * (_lib.INT4_GROUPS_PER_WG * 2)
                table = torch.cat([table4[:, :3], zcol.unsqueeze(1), table4[:, 3:]], dim=1)
            else:
                table, owner, local = tile_table(rows, bm, bn) if fp8 else item_table(rows, plan.group)
            blocks.append(table)
            owners.append(row_slot[owner])
            order.append(first[owner] * (1 << 32) + local)
        if copy_rows:
            c = torch.tensor([(r + (0,))[:5] for r in copy_rows], dtype=torch.int64)     # mi, slot, dst, bytes, src offset
            counts = (c[:, 3] + _COPY - 1) // _COPY
            owner = torch.repeat_interleave(torch.arange(len(copy_rows)), counts)
            start = torch.cumsum(counts, 0) - counts
            local = torch.arange(int(counts.sum()), dtype=torch.int64) - start[owner]
            d = c[owner]
            nb = torch.clamp(d[:, 3] - local * _COPY, max=_COPY)
            zero = torch.zeros_like(nb)
            src, dst = d[:, 4] + local * _COPY, d[:, 2] + local * _COPY
            if fp8:
                blocks.append(torch.stack([src, dst, zero, nb, zero, torch.full_like(nb, _lib.BUCKET_COPY_MARK), zero, zero], dim=1))
            elif asym:
                blocks.append(torch.stack([src, dst, zero, zero, -nb], dim=1))
            else:
                blocks.append(torch.stack([src, dst, zero, -nb], dim=1))
            owners.append(d[:, 1])
            order.append(d[:, 0] * (1 << 32) + local)
        if blocks:
            perm = torch.argsort(torch.cat(order), stable=True)
            table = torch.cat(blocks, dim=0)[perm].contiguous()
            owner_all = torch.cat(owners)[perm]
            assert table.shape[1] == width
            plan.n_items = table.shape[0]
            if fp8:
                # FP8 tiles whose code rows do not start on 64-byte boundaries of the buffer (an earlier tensor of the bucket
                # left them there: back-to-back packing decides every address) go to the launch with plain stores, where
                # the two tiles that share each 128-byte line get their halves merged in the L2
                off_lines = (table[:, 5] != _lib.BUCKET_COPY_MARK) & (((table[:, 1] | table[:, 7]) & 63) != 0)
                if bool(off_lines.any()):
                    plan.table_off_lines = ResolvedTable(table[off_lines].contiguous(), owner_all[off_lines], const_slot + 1, device)
                    table, owner_all = table[~off_lines].contiguous(), owner_all[~off_lines]
            plan.table = ResolvedTable(table, owner_all, const_slot + 1, device) if table.shape[0] else None
            plan.slot_src = np.asarray(slot_src, dtype=np.int64)
            plan.align = np.asarray(align, dtype=np.int64)
        if zp_entries:
            zrows, zstart, plan.zp_words = zero_point_rows(zp_entries)
            plan.zp_rows, plan.zp_start = zrows.to(device), zstart.to(device)
        # The layout holds no address of an input and no reference to one: it serves every later bucket with the same
        # names, shapes, strides and dtypes wherever its tensors live, and it keeps no weight alive.
        return plan

    def _resolve(self, plan: _Layout, ptrs) -> bool:
        """The bucket's tensors are not where the resolved table says: upload their addresses (8 bytes each, through
        pinned staging) and let the GPU add them to the template.  -> False when an input the kernels need aligned
        is not (the cached routing does not apply to these tensors)."""
        arr = np.asarray(ptrs, dtype=np.int64)
        bases = arr[plan.slot_src]
        if np.any(bases & plan.align):
            return False
        bases = np.append(bases, plan.const_base)
        for table in (plan.table, plan.table_off_lines):
            if table is not None:
                table.resolve(bases, tag=ptrs)
        self.resolves += 1
        return True

    # ------------------------------------------------------------------ run

    def convert(self, params, out: torch.Tensor | None = None, bucket_id=None) -> FlattenedBucket:
        """``bucket_id`` (any hashable, e.g. the bucket's index in the weight-sync loop) is a promise that every call
        with this id presents the same names, shapes, strides and dtypes; the layout is then found by the id alone
        (without it, by the full identity of the bucket - names, shapes, dtypes, strides: under a microsecond per tensor).  Where the tensors live may change
        from call to call: a moved bucket costs one upload of its addresses and one small launch."""
        params = [(mn, conv if type(conv) is list else list(conv)) for mn, conv in params]
        ptrs = [t.data_ptr() for _, conv in params for _, t in conv]
        if not ptrs:
            return flatten_named_tensors([])
        if bucket_id is not None:
            key = ("id", bucket_id, ue8m0_requant_enabled())
        else:
            key = (self._key(params), self._config_key, self.transform_ue8m0, ue8m0_requant_enabled())
        plan = self._layouts.get(key)
        if plan is not None and plan.n_tensors != len(ptrs):
            plan = None                                  # not the bucket this id stood for
        for _ in range(2):
            if plan is None:
                plan = self._build(params)
                self._layouts[key] = plan
                while len(self._layouts) > self._max:
                    self._layouts.popitem(last=False)
            else:
                self._layouts.move_to_end(key)
            if plan.fallback:
                # back-to-back packing puts a tensor at an offset that is not a multiple of its element size:
                # the per-parameter loop and a plain concatenation, exactly as the reference builds the buffer
                flat = flatten_named_tensors(per_param_loop(self.args, params, self.config, self.transform_ue8m0))
                if out is None:
                    return flat
                self._check_out(out, plan.total_bytes, plan.device)
                out[:plan.total_bytes].copy_(flat.get_flattened_tensor())
                return FlattenedBucket(out[:plan.total_bytes], flat.get_metadata(), flat.launches + 1)
            if not plan.n_items or ptrs == (plan.table or plan.table_off_lines).resolved_for or self._resolve(plan, ptrs):
                break
            plan = None                                  # an input lost the alignment the cached routing relied on
        device = plan.device
        if out is None:
            out = torch.empty(plan.total_bytes, dtype=torch.uint8, device=device)
        else:
            self._check_out(out, plan.total_bytes, device)
        launches = 0
        if plan.n_items:
            lib = _lib.load()
            if self.time_kernels:
                ev = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                ev[0].record(torch.cuda.current_stream(device))
            with torch.cuda.device(device):
                if plan.kind == "fp8":
                    rc = 0
                    if plan.table is not None:
                        rc = lib.wq_fp8_bucket_convert(plan.table.items.data_ptr(), plan.table.n_items, out.data_ptr(),
                                                       plan.block[0], plan.block[1], _lib.FP8_MODE_TRITON, _lib.stream_ptr(device))
                    if rc == 0 and plan.table_off_lines is not None:
                        rc = lib.wq_fp8_bucket_convert_rows_off_lines(
                            plan.table_off_lines.items.data_ptr(), plan.table_off_lines.n_items, out.data_ptr(),
                            plan.block[0], plan.block[1], _lib.FP8_MODE_TRITON, _lib.stream_ptr(device))
                        launches += plan.table is not None
                elif plan.kind == "int4_asym":
                    # the pack kernel leaves every group's zero point in a scratch buffer; a second launch packs them
                    # eight rows to a word into their place in the bucket
                    zero = torch.empty(max(plan.zero_bytes, 16), dtype=torch.uint8, device=device)
                    rc = lib.wq_int4_group_quant_pack_asym_items(plan.table.items.data_ptr(), plan.n_items, out.data_ptr(),
                                                                 zero.data_ptr(), plan.group, _lib.stream_ptr(device))
                    if rc == 0 and plan.n_zp:
                        rc = lib.wq_int4_zero_point_pack_grouped(plan.zp_rows.data_ptr(), plan.zp_start.data_ptr(), plan.n_zp,
                                                                 plan.zp_words, zero.data_ptr(), out.data_ptr(),
                                                                 _lib.stream_ptr(device))
                        launches += 1
                else:
                    rc = lib.wq_int4_bucket_convert(plan.table.items.data_ptr(), plan.n_items, out.data_ptr(), plan.group,
                                                    _lib.stream_ptr(device))
            _lib.check(rc, "BucketConverter.convert")
            launches += 1
            if self.time_kernels:
                ev[1].record(torch.cuda.current_stream(device))
                self.kernel_events.append(ev)
        if plan.late_copies:
            launches += self._late(plan, params, out)
        return FlattenedBucket(out[:plan.total_bytes], plan.metadata, launches)

    @staticmethod
    def _check_out(out, total_bytes, device) -> None:
        if out.dtype != torch.uint8 or out.dim() != 1 or out.numel() < total_bytes or not out.is_contiguous() \
                or out.device != device or out.data_ptr() % 128:
            raise ValueError(f"out must be a contiguous 128-byte aligned uint8 vector of at least {total_bytes} bytes on {device}")

    def kernel_ms(self) -> float:
        """Sum of the launch times recorded while ``time_kernels`` was set (call after a synchronize); clears the list."""
        total = sum(a.elapsed_time(b) for a, b in self.kernel_events)
        self.kernel_events = []
        return total

    def _late(self, plan, params, out) -> int:
        """Tensors outside the one-launch kernels: per-tensor functions, then one copy each."""
        n, cache = 0, {}
        for mi, pi, ci, out_name in plan.late_copies:
            m = plan.metadata[mi]
            mn, conv = params[pi]
            name, t = conv[ci]
            if out_name is None:
                src = t
            else:
                if (pi, ci) not in cache:
                    cache[(pi, ci)] = dict(quantize_params(self.args, mn, [(name, t)], self.config, self.transform_ue8m0))
                    n += 1
                src = cache[(pi, ci)][out_name]
            out[m.start_idx:m.end_idx].copy_(src.detach().to(out.device).contiguous().flatten().view(torch.uint8))
            n += 1
        return n


def quantize_bucket(args, params, quantization_config, transform_ue8m0: bool = True,
                    converter: BucketConverter | None = None) -> FlattenedBucket:
    """One-call form: ``params`` = ``[(megatron_name, [(hf_name, tensor), ...]), ...]`` for a whole bucket.  Pass the
    same ``converter`` on every sync to reuse its cached tables."""
    conv = converter or BucketConverter(args, quantization_config, transform_ue8m0)
    return conv.convert(params)


def per_param_loop(args, params, quantization_config, transform_ue8m0: bool = True):
    """The loop this module replaces, on the per-tensor functions: -> [(hf_name, tensor), ...] in bucket order."""
    outs = []
    for mn, conv in params:
        outs.extend(quantize_params(args, mn, list(conv), quantization_config, transform_ue8m0))
    return outs
