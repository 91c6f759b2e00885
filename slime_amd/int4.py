"""Group-wise INT4 weight quantisation and packing on MI355X.

Mirrors, name for name, the functions of tools/convert_hf_to_int4_direct.py:32-153 (identical copies live
in slime/backends/megatron_utils/megatron_to_hf/processors/quantizer_compressed_tensors.py:137-265) and
the extension entry point fake_int4_quant_cuda(x, block_size, sym) of
slime/backends/megatron_utils/kernels/int4_qat/fake_int4_quant_cuda.cu:327-378.

``pack_layer`` on a bf16 weight runs ONE fused HIP kernel (amax or min/max, scale, divide, round, nibble pack),
symmetric or asymmetric.  The reference's intermediate dequantise / re-quantise steps map every integer
code back to itself for all reachable (code, bf16 scale) pairs - the test-suite re-proves this by
exhaustion - so they are not executed there; where they are not the identity (scales of 2^121 and above,
asymmetric codes above 17) the kernels run them literally.  Other dtypes, strides and group sizes run the HIP
fake-quant kernel and then the reference's own chain of tensor ops on the GPU.
"""

from __future__ import annotations

import math
import threading
from collections import OrderedDict
from typing import Sequence

import torch

from . import _lib, arith


def _dtype_sel(t: torch.Tensor, what: str) -> int:
    if t.dtype == torch.bfloat16:
        return _lib.DTYPE_BF16
    if t.dtype == torch.float32:
        return _lib.DTYPE_F32
    if t.dtype == torch.float64:
        return _lib.DTYPE_F64
    # the reference dispatches on float, double and bfloat16 (fake_int4_quant_cuda.cu:352-354) and raises for the rest
    names = {torch.float16: "Half", torch.int8: "Char", torch.uint8: "Byte", torch.int16: "Short", torch.int32: "Int",
             torch.int64: "Long", torch.bool: "Bool"}
    raise RuntimeError(f'"{what}" not implemented for \'{names.get(t.dtype, str(t.dtype).replace("torch.", ""))}\'')


def fake_int4_quant_cuda(x: torch.Tensor, block_size: Sequence[int], sym: bool):
    """-> (q, scale, zero): q has x's shape and dtype and holds the integer codes as floats; scale and
    zero are [ceil(M/bm), ceil(N/bn)] in x's dtype.  Errors are RuntimeError, as TORCH_CHECK raises
    (fake_int4_quant_cuda.cu:333-344)."""
    if x.dim() != 2:
        raise RuntimeError("Input must be 2D")
    if not x.is_cuda:
        raise RuntimeError("Input must be on the GPU")
    bm, bn = int(block_size[0]), int(block_size[1])
    if bm <= 0 or bn <= 0:
        raise RuntimeError(f"Block sizes must be positive, got block_m={bm}, block_n={bn}")
    if (bm * bn) % 32 != 0:
        raise RuntimeError(f"block_m * block_n ({bm * bn}) must be divisible by 32. But got a {bm}x{bn} block.")
    sel = _dtype_sel(x, "fake_int4_quant_cuda")
    M, N = x.shape
    q = torch.empty((M, N), dtype=x.dtype, device=x.device)
    scale = torch.empty((-(-M // bm), -(-N // bn)), dtype=x.dtype, device=x.device)
    zero = torch.empty_like(scale)
    with torch.cuda.device(x.device):
        rc = _lib.load().wq_int4_fake_quant(x.data_ptr(), sel, M, N, x.stride(0), x.stride(1), bm, bn, int(bool(sym)),
                                            q.data_ptr(), scale.data_ptr(), zero.data_ptr(), _lib.stream_ptr(x.device))
    _lib.check(rc, "fake_int4_quant_cuda")
    return q, scale, zero


def pack_to_int32(value: torch.Tensor, num_bits: int, packed_dim: int = 1, sym: bool = False) -> torch.Tensor:
    """Pack ``32 // num_bits`` integers per int32 along ``packed_dim``; element j of a word sits at bits
    [j*num_bits, (j+1)*num_bits).  ``sym`` adds the offset 2**(num_bits-1) first.
    (tools/convert_hf_to_int4_direct.py:32-75; pure integer tensor ops on value's device.)"""
    if num_bits > 8:
        raise ValueError("Packing is only supported for less than 8 bits")
    if num_bits < 1:
        raise ValueError(f"num_bits must be at least 1, got {num_bits}")
    if sym:
        value = (value + (1 << (num_bits - 1))).to(torch.uint8)
    per_word = 32 // num_bits
    if packed_dim == 0:
        value = value.transpose(0, 1)
    rows, cols = value.shape
    n_words = math.ceil(cols / per_word)
    if n_words * per_word != cols:
        value = torch.nn.functional.pad(value, (0, n_words * per_word - cols))
    shifts = torch.arange(per_word, device=value.device, dtype=torch.int32) * num_bits
    words = (value.view(rows, n_words, per_word).to(torch.int32) << shifts).sum(dim=2, dtype=torch.int32)
    return words.transpose(0, 1) if packed_dim == 0 else words


def round_to_quantized_type_dtype(tensor: torch.Tensor, dtype: torch.dtype, cast_to_original_dtype: bool = False):
    """clamp to dtype's integer range, round half to even, cast (convert_hf_to_int4_direct.py:78-88)."""
    lim = torch.iinfo(dtype)
    out = torch.round(torch.clamp(tensor, lim.min, lim.max)).to(dtype)
    return out.to(tensor.dtype) if cast_to_original_dtype else out


@torch.no_grad()
def quantize(x: torch.Tensor, scale: torch.Tensor, zero_point, dtype: torch.dtype = torch.int8) -> torch.Tensor:
    """x / scale (+ zero_point) per group of x.shape[-1] // scale.shape[-1] columns, clamped, rounded and
    cast to ``dtype`` (convert_hf_to_int4_direct.py:91-120)."""
    group = x.shape[-1] // scale.shape[-1]
    scaled = x.unflatten(-1, (math.ceil(x.shape[-1] / group), group)) / scale.unsqueeze(-1)
    if zero_point is not None:
        scaled += zero_point.unsqueeze(-1).to(x.dtype)
    return round_to_quantized_type_dtype(scaled, dtype).flatten(start_dim=-2).to(dtype)


def _check_pack_input(weight: torch.Tensor, group_size: int, what: str) -> None:
    if weight.dim() != 2:
        raise RuntimeError(f"{what}: expected a 2-D weight")
    _lib.require_gpu(weight, what)
    if group_size <= 0 or weight.shape[1] % group_size != 0:
        # the reference fails in .view(M, 1, N // group_size, group_size)
        raise RuntimeError(f"{what}: shape '{[weight.shape[0], 1, weight.shape[1] // max(group_size, 1), group_size]}' "
                           f"is invalid for input of size {weight.numel()}")
    if group_size % 32 != 0:
        raise RuntimeError(f"block_m * block_n ({group_size}) must be divisible by 32. But got a 1x{group_size} block.")


def _pack_zero_points_awq(zp: torch.Tensor) -> torch.Tensor:
    """[M, G] zero points -> int32 [G, M/8]: transposed, eight row-consecutive values per word in the nibble
    order 0,4,1,5,2,6,3,7 (convert_hf_to_int4_direct.py:134-141)."""
    z = zp.t().contiguous().to(torch.float32).to(torch.int32)
    awq_order = torch.tensor([0, 4, 1, 5, 2, 6, 3, 7], device=z.device) * 4
    return (z.reshape(-1, z.shape[1] // 8, 8) << awq_order).sum(dim=-1).to(torch.int32)


def pack_layer(weight: torch.Tensor, group_size: int, sym: bool = True):
    """-> (weight_packed int32 [M, N/8], weight_scale [M, N/group_size] in weight dtype,
    packed_zero_point int32 [N/group_size, M/8] or None).  convert_hf_to_int4_direct.py:123-153."""
    _check_pack_input(weight, group_size, "pack_layer")
    M, N = weight.shape
    if sym and weight.dtype == torch.bfloat16 and weight.stride(1) == 1:
        packed = torch.empty((M, N // 8), dtype=torch.int32, device=weight.device)
        scale = torch.empty((M, N // group_size), dtype=torch.bfloat16, device=weight.device)
        if M and N:
            with torch.cuda.device(weight.device):
                rc = _lib.load().wq_int4_group_quant_pack(weight.data_ptr(), M, N, weight.stride(0), int(group_size),
                                                          packed.data_ptr(), scale.data_ptr(),
                                                          _lib.stream_ptr(weight.device))
            _lib.check(rc, "pack_layer")
        return packed, scale, None

    if (not sym and weight.dtype == torch.bfloat16 and weight.stride(1) == 1 and group_size in (32, 64, 128)
            and weight.stride(0) % 8 == 0 and weight.data_ptr() % 16 == 0 and M and N):
        # fused asymmetric quantise + pack; only the (small) zero-point tensor goes through tensor ops
        packed = torch.empty((M, N // 8), dtype=torch.int32, device=weight.device)
        scale = torch.empty((M, N // group_size), dtype=torch.bfloat16, device=weight.device)
        zp = torch.empty_like(scale)
        with torch.cuda.device(weight.device):
            rc = _lib.load().wq_int4_group_quant_pack_asym(weight.data_ptr(), M, N, weight.stride(0), int(group_size),
                                                           packed.data_ptr(), scale.data_ptr(), zp.data_ptr(),
                                                           _lib.stream_ptr(weight.device))
        _lib.check(rc, "pack_layer")
        return packed, scale, _pack_zero_points_awq(zp)

    # general form: HIP fake-quant kernel, then the reference's tensor-op chain on the GPU
    G = N // group_size
    q, scale, zp = fake_int4_quant_cuda(weight, (1, group_size), sym)
    q = q.view(M, 1, G, group_size)
    scale = scale.view(M, 1, G, 1)
    zp = zp.view(M, 1, G, 1)
    deq = (q * scale if sym else (q - zp) * scale).view(M, N)
    scale = scale.view(M, -1).contiguous()
    if sym:
        zp = packed_zp = None
    else:
        zp = zp.view(M, -1)
        packed_zp = _pack_zero_points_awq(zp)
    codes = quantize(deq, scale, zp, torch.int8 if sym else torch.uint8)
    return pack_to_int32(codes, 4, sym=sym), scale, packed_zp


_ITEM_TABLE_MIN_TENSORS = 64     # plans with at least this many tensors pre-resolve every work item on the host


def item_table(rows, group: int):
    """One descriptor per work item of WQ_INT4_GROUPS_PER_WG groups from per-tensor rows ``[x, packed, scale, n_groups]``
    (addresses, or byte offsets for the bucket launches).  -> (int64 [items, 4] in tensor order; owner and local index
    per item)."""
    per = _lib.INT4_GROUPS_PER_WG
    desc = torch.as_tensor(rows, dtype=torch.int64).reshape(-1, 4)
    counts = (desc[:, 3] + per - 1) // per
    owner = torch.repeat_interleave(torch.arange(desc.shape[0]), counts)
    local = torch.arange(int(counts.sum()), dtype=torch.int64) - (torch.cumsum(counts, 0) - counts)[owner]
    d = desc[owner]
    table = torch.stack([d[:, 0] + local * (per * group * 2), d[:, 1] + local * (per * group // 8 * 4),
                         d[:, 2] + local * (per * 2), torch.clamp(d[:, 3] - local * per, max=per)], dim=1)
    return table, owner, local


def zero_point_rows(entries):
    """Descriptor rows and prefix sums for ``wq_int4_zero_point_pack_grouped`` from ``(zero, out, M, G)`` tuples
    (addresses or byte offsets).  -> (int64 [n, 4], int64 [n + 1], total words)."""
    rows = torch.tensor([[z, o, M, G] for z, o, M, G in entries], dtype=torch.int64).reshape(-1, 4)
    words = rows[:, 3] * (rows[:, 2] // 8)
    start = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(words, 0)])
    return rows, start, int(start[-1])


class Int4PackPlan:
    """Quantise+pack of a fixed list of contiguous bf16 weights with one launch per ``run()`` (symmetric) or two
    (asymmetric: the pack kernel, then one kernel that packs every tensor's zero points in AWQ order).

    ``outputs`` holds ``(weight_packed int32 [M,N/8], weight_scale bf16 [M,N/group])`` - plus
    ``packed_zero_point int32 [N/group, M/8]`` when ``sym`` is false - views into the plan's flat buffers, in input
    order: what ``pack_layer(w, group_size, sym)`` returns for each weight."""

    def __init__(self, weights: Sequence[torch.Tensor], group_size: int = 128, sym: bool = True):
        if not weights:
            raise ValueError("Int4PackPlan: empty weight list")
        if group_size not in (32, 64, 128):
            raise ValueError("Int4PackPlan: group_size must be 32, 64 or 128")
        self.group, self.sym = int(group_size), bool(sym)
        self.device = weights[0].device
        self.weights = list(weights)
        p_off, s_off, z_off, p_total, s_total, z_total = [], [], [], 0, 0, 0
        for w in self.weights:
            _check_pack_input(w, self.group, "Int4PackPlan")
            if w.dtype != torch.bfloat16 or not w.is_contiguous() or w.data_ptr() % 16:
                raise ValueError("Int4PackPlan: weights must be contiguous, 16-byte aligned bfloat16")
            M, N = w.shape
            if not self.sym and M % 8:
                # zero points are packed eight ROWS to a word (convert_hf_to_int4_direct.py:134-141); pack_layer itself
                # takes such a weight through the reference's reshape, whatever that yields or raises
                raise ValueError(f"Int4PackPlan(sym=False): {M} rows are not a multiple of 8")
            p_off.append(p_total)
            s_off.append(s_total)
            z_off.append(z_total)
            p_total += (M * N // 8 + 63) // 64 * 64
            s_total += (M * N // self.group + 127) // 128 * 128
            z_total += ((N // self.group) * (M // 8) + 63) // 64 * 64
        self.flat_packed = torch.empty(max(p_total, 1), dtype=torch.int32, device=self.device)
        self.flat_scale = torch.empty(max(s_total, 1), dtype=torch.bfloat16, device=self.device)
        rows, starts, work = [], [0], 0
        self.outputs = []
        if not self.sym:
            self._zero = torch.empty(max(s_total, 1), dtype=torch.bfloat16, device=self.device)     # [M, N/group] per tensor
            self.flat_zp = torch.empty(max(z_total, 1), dtype=torch.int32, device=self.device)
        zp_entries = []
        for w, po, so, zo in zip(self.weights, p_off, s_off, z_off):
            M, N = w.shape
            n_groups = M * N // self.group
            packed = self.flat_packed[po:po + M * N // 8].view(M, N // 8)
            scale = self.flat_scale[so:so + n_groups].view(M, N // self.group)
            if self.sym:
                self.outputs.append((packed, scale))
                rows.append([w.data_ptr(), packed.data_ptr(), scale.data_ptr(), n_groups])
            else:
                G = N // self.group
                zp = self.flat_zp[zo:zo + G * (M // 8)].view(G, M // 8)
                zero = self._zero[so:so + n_groups]
                self.outputs.append((packed, scale, zp))
                rows.append([w.data_ptr(), packed.data_ptr(), scale.data_ptr(), zero.data_ptr(), n_groups])
                zp_entries.append((zero.data_ptr(), zp.data_ptr(), M, G))
            work += -(-n_groups // _lib.INT4_GROUPS_PER_WG)
            starts.append(work)
        self.total_work = work
        self.bf16_bytes = sum(2 * w.numel() for w in self.weights)
        self._items = None
        if not self.sym:
            # one descriptor per work item: x, packed, scale, zero advance with the item; n_groups is what is left
            per = _lib.INT4_GROUPS_PER_WG
            desc = torch.tensor(rows, dtype=torch.int64)
            start = torch.tensor(starts, dtype=torch.int64)
            owner = torch.repeat_interleave(torch.arange(len(rows)), start[1:] - start[:-1])
            local = torch.arange(work, dtype=torch.int64) - start[owner]
            d = desc[owner]
            items = torch.stack([d[:, 0] + local * (per * self.group * 2), d[:, 1] + local * (per * self.group // 8 * 4),
                                 d[:, 2] + local * (per * 2), d[:, 3] + local * (per * 2),
                                 torch.clamp(d[:, 4] - local * per, max=per)], dim=1)
            self._items = items.contiguous().to(self.device)
            zrows, zstart, self._zp_words = zero_point_rows(zp_entries)
            self._zp_rows, self._zp_start = zrows.to(self.device), zstart.to(self.device)
        elif len(rows) >= _ITEM_TABLE_MIN_TENSORS:
            # Many small tensors (the experts of a model): one pre-resolved descriptor per work item (32 bytes per 16 KiB
            # of weights), so that the kernel needs a single scalar load instead of a search through the per-tensor
            # prefix sums.  A handful of tensors keeps the search.
            items, _, _ = item_table(rows, self.group)
            self._items = items.contiguous().to(self.device)
        else:
            self._descs = torch.tensor(rows, dtype=torch.int64).to(self.device)
            self._starts = torch.tensor(starts, dtype=torch.int64).to(self.device)

    def run(self):
        lib = _lib.load()
        st = _lib.stream_ptr(self.device)
        with torch.cuda.device(self.device):
            if not self.sym:
                rc = lib.wq_int4_group_quant_pack_asym_items(self._items.data_ptr(), self.total_work, None, None, self.group, st)
                if rc == 0:
                    rc = lib.wq_int4_zero_point_pack_grouped(self._zp_rows.data_ptr(), self._zp_start.data_ptr(),
                                                             len(self.weights), self._zp_words, None, None, st)
            elif self._items is not None:
                rc = lib.wq_int4_group_quant_pack_items(self._items.data_ptr(), self.total_work, self.group, st)
            else:
                rc = lib.wq_int4_group_quant_pack_grouped(self._descs.data_ptr(), self._starts.data_ptr(),
                                                          len(self.weights), self.total_work, self.group, st)
        _lib.check(rc, "Int4PackPlan.run")
        return self.outputs


# ------------------------------------------------------------------------------------ inverse and QAT forward


_SCALE_DTYPES = {torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_F16, torch.float32: _lib.DTYPE_F32}


def dequantize_int4(weight_packed: torch.Tensor, weight_scale: torch.Tensor, weight_shape, group_size: int) -> torch.Tensor:
    """pack-quantized INT4 -> bf16: ``((nibble - 8).to(f32) * scale.to(f32)).to(bf16)`` with the scale of each
    ``group_size`` columns, the arithmetic of ``_dequantize_tensor`` in
    tools/convert_k2_thinking_int4_to_bf16.py:55-84 (its unpacking step is ``compressed_tensors.unpack_from_int32``:
    nibble j of a word at bits [4j, 4j+4), offset 8, rows cut to their length).  ``weight_shape`` is the
    ``.weight_shape`` tensor or a tuple.  As there, the scale may have any floating dtype (bf16, fp16 and fp32 are read
    as stored, others are converted to fp32 first) and ``group_size <= 0`` means one scale per weight element.  bf16
    scales with groups of a multiple of 8 take the bandwidth-tuned kernel."""
    _lib.require_gpu(weight_packed, "dequantize_int4")
    shape = tuple(int(v) for v in (weight_shape.view(-1).tolist() if isinstance(weight_shape, torch.Tensor) else weight_shape))
    if len(shape) != 2:
        raise ValueError(f"dequantize_int4: expected a 2-D weight shape, got {shape}")
    M, N = shape
    if weight_packed.dtype != torch.int32 or tuple(weight_packed.shape) != (M, -(-N // 8)):
        raise ValueError(f"dequantize_int4: weight_packed {tuple(weight_packed.shape)} {weight_packed.dtype} does not "
                         f"match shape {shape}")
    group = int(group_size) if group_size > 0 else 1
    if N % group != 0:
        raise ValueError(f"Scale shape {tuple(weight_scale.shape)} incompatible with weight shape {shape}")
    scale = weight_scale.unsqueeze(1) if (weight_scale.dim() == 1 and group_size > 0) else weight_scale
    if scale.numel() != M * (N // group):
        raise ValueError(f"Scale shape {tuple(weight_scale.shape)} incompatible with weight shape {shape}")
    if scale.dtype not in _SCALE_DTYPES:
        scale = scale.to(torch.float32)
    scale = scale.contiguous()
    packed = weight_packed.contiguous()
    y = torch.empty((M, N), dtype=torch.bfloat16, device=packed.device)
    if M and N:
        lib = _lib.load()
        with torch.cuda.device(packed.device):
            if scale.dtype == torch.bfloat16 and group % 8 == 0:
                rc = lib.wq_int4_dequant(packed.data_ptr(), scale.data_ptr(), y.data_ptr(), M, N, group,
                                         _lib.stream_ptr(packed.device))
            else:
                rc = lib.wq_int4_dequant_any(packed.data_ptr(), scale.data_ptr(), _SCALE_DTYPES[scale.dtype], y.data_ptr(),
                                             M, N, group, _lib.stream_ptr(packed.device))
        _lib.check(rc, "dequantize_int4")
    return y


class Int4DequantPlan:
    """``dequantize_int4`` over a fixed list of (weight_packed, weight_scale, shape) triples with one launch per
    ``run()``; ``outputs`` holds bf16 ``[M, N]`` views into one flat buffer (``flat_y``), in input order.  The group
    size must be a power of two (32, 64, 128 ...)."""

    def __init__(self, packeds: Sequence[torch.Tensor], scales: Sequence[torch.Tensor], shapes, group_size: int):
        if not packeds or len(packeds) != len(scales) or len(packeds) != len(shapes):
            raise ValueError("Int4DequantPlan: need equally many packed tensors, scales and shapes")
        per = _lib.INT4_DEQ_WORDS_PER_ITEM
        if group_size < 8 or group_size & (group_size - 1) or group_size > 8 * per:
            raise ValueError(f"Int4DequantPlan: group_size {group_size} must be a power of two in [8, {8 * per}]")
        self.group = int(group_size)
        self.device = packeds[0].device
        self.packeds, self.scales = [], []
        y_off, total = [], 0
        shapes = [tuple(int(v) for v in (sh.view(-1).tolist() if isinstance(sh, torch.Tensor) else sh)) for sh in shapes]
        for p, sc, (M, N) in zip(packeds, scales, shapes):
            _lib.require_gpu(p, "Int4DequantPlan")
            if p.dtype != torch.int32 or tuple(p.shape) != (M, N // 8) or N % self.group or sc.dtype != torch.bfloat16 \
                    or sc.numel() != M * (N // self.group) or p.device != self.device or sc.device != self.device:
                raise ValueError(f"Int4DequantPlan: packed {tuple(p.shape)} {p.dtype} / scale {tuple(sc.shape)} {sc.dtype} "
                                 f"do not describe a [{M}, {N}] weight with groups of {self.group}")
            if not p.is_contiguous() or not sc.is_contiguous():
                # a plan reads its inputs again on every run: a silent copy would freeze them at construction time
                raise ValueError("Int4DequantPlan: packed weights and scales must be contiguous")
            self.packeds.append(p)
            self.scales.append(sc)
            y_off.append(total)
            total += (M * N + 127) // 128 * 128
        self.flat_y = torch.empty(max(total, 1), dtype=torch.bfloat16, device=self.device)
        self.outputs = [self.flat_y[o:o + M * N].view(M, N) for o, (M, N) in zip(y_off, shapes)]
        n_words = torch.tensor([M * N // 8 for M, N in shapes], dtype=torch.int64)
        counts = (n_words + per - 1) // per
        start = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(counts, 0)])
        owner = torch.repeat_interleave(torch.arange(len(shapes)), counts)
        local = torch.arange(int(start[-1]), dtype=torch.int64) - start[owner]
        pbase = torch.tensor([p.data_ptr() for p in self.packeds], dtype=torch.int64)
        sbase = torch.tensor([sc.data_ptr() for sc in self.scales], dtype=torch.int64)
        ybase = torch.tensor([y.data_ptr() for y in self.outputs], dtype=torch.int64)
        items = torch.stack([pbase[owner] + local * (per * 4), sbase[owner] + local * (per * 8 // self.group * 2),
                             ybase[owner] + local * (per * 16), torch.clamp(n_words[owner] - local * per, max=per)], dim=1)
        self.total_items = int(start[-1])
        self._items = items.contiguous().to(self.device)
        self.bf16_bytes = 2 * sum(M * N for M, N in shapes)

    def run(self):
        with torch.cuda.device(self.device):
            rc = _lib.load().wq_int4_dequant_items(self._items.data_ptr(), self.total_items, self.group,
                                                   _lib.stream_ptr(self.device))
        _lib.check(rc, "Int4DequantPlan.run")
        return self.outputs


class _FakeInt4QuantizationSTE(torch.autograd.Function):
    """Quantise-dequantise forward, identity backward (docker/patch/latest/megatron.patch:212-255)."""

    @staticmethod
    def forward(ctx, x, group_size):
        _lib.require_gpu(x, "fake_int4_quantization_ste")
        m, n = x.shape
        if x.dtype == torch.bfloat16 and group_size in (32, 64, 128) and n % group_size == 0:
            xc = x.contiguous()
            y = torch.empty_like(xc)
            if m and n:
                with torch.cuda.device(x.device):
                    rc = _lib.load().wq_int4_fake_quant_ste(xc.data_ptr(), y.data_ptr(), m, n, int(group_size),
                                                            arith.div7_rule(), _lib.stream_ptr(x.device))
                _lib.check(rc, "fake_int4_quantization_ste")
            return y
        # ragged widths, other group sizes or dtypes: the reference's own tensor ops, on the GPU
        n_pad = -(-n // group_size) * group_size
        xp = torch.zeros((m, n_pad), dtype=x.dtype, device=x.device)
        xp[:, :n] = x
        view = xp.view(m, 1, n_pad // group_size, group_size)
        amax = view.abs().float().amax(dim=(1, 3), keepdim=True)
        # `amax / 7` is torch's GPU evaluation (a reciprocal multiply); a tensor divisor forces the IEEE division
        seven = 7 if arith.get_torch_arithmetic() == "device" else torch.full((), 7.0, device=x.device)
        scale = (amax / seven).clamp(min=1e-5)
        deq = torch.round(view / scale).clamp(-7, 7) * scale
        return deq.view_as(xp)[:, :n].contiguous().to(x.dtype)

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None


def fake_int4_quantization_ste(x: torch.Tensor, group_size: int) -> torch.Tensor:
    out = _FakeInt4QuantizationSTE.apply(x, group_size)
    if hasattr(x, "main_grad"):
        out.main_grad = x.main_grad
    return out


_STE_TABLES: OrderedDict = OrderedDict()
_STE_LOCK = threading.Lock()


def _ste_table(xs, group_size):
    """Per-item table of the one-launch STE forward for these weights (y as offsets into one output buffer), cached on
    the addresses and shapes of the weights: a layer that calls again with the same parameters builds nothing."""
    device = xs[0].device
    key = (group_size, device.index, tuple((x.data_ptr(), x.shape[0], x.shape[1]) for x in xs))
    with _STE_LOCK:
        entry = _STE_TABLES.get(key)
        if entry is not None:
            _STE_TABLES.move_to_end(key)
            return entry
    per = _lib.INT4_GROUPS_PER_WG
    rows, offs, off = [], [], 0
    for x in xs:
        rows.append([x.data_ptr(), off, x.numel() // group_size])
        offs.append(off // 2)
        off += (2 * x.numel() + 15) // 16 * 16
    desc = torch.tensor(rows, dtype=torch.int64)
    counts = (desc[:, 2] + per - 1) // per
    owner = torch.repeat_interleave(torch.arange(len(rows)), counts)
    local = torch.arange(int(counts.sum()), dtype=torch.int64) - (torch.cumsum(counts, 0) - counts)[owner]
    d = desc[owner]
    step = per * group_size * 2
    items = torch.stack([d[:, 0] + local * step, d[:, 1] + local * step, torch.clamp(d[:, 2] - local * per, max=per)], dim=1)
    entry = (items.contiguous().to(device), items.shape[0], offs, off // 2)
    with _STE_LOCK:
        _STE_TABLES[key] = entry
        while len(_STE_TABLES) > 1024:
            _STE_TABLES.popitem(last=False)
    return entry


class Int4StePlan:
    """The QAT quantise-dequantise forward over a fixed list of contiguous bf16 weights with one launch per ``run()``;
    ``outputs`` are views into the plan's flat buffer, in input order (no autograd: the inference-side / benchmark
    form of ``fake_int4_quantization_ste_many``)."""

    def __init__(self, weights: Sequence[torch.Tensor], group_size: int = 128):
        if not weights or group_size not in (32, 64, 128):
            raise ValueError("Int4StePlan: need at least one weight and a group size of 32, 64 or 128")
        for w in weights:
            _lib.require_gpu(w, "Int4StePlan")
            if w.dim() != 2 or w.dtype != torch.bfloat16 or not w.is_contiguous() or w.data_ptr() % 16 or not w.numel() \
                    or w.shape[1] % group_size:
                raise ValueError("Int4StePlan: weights must be non-empty contiguous 16-byte aligned bfloat16 matrices "
                                 "whose rows are whole groups")
        self.group, self.device, self.weights = int(group_size), weights[0].device, list(weights)
        self._items, self.n_items, offs, total = _ste_table(self.weights, self.group)
        self.flat_y = torch.empty(total, dtype=torch.bfloat16, device=self.device)
        self.outputs = [self.flat_y[o:o + w.numel()].view(w.shape) for o, w in zip(offs, self.weights)]
        self.bf16_bytes = sum(2 * w.numel() for w in self.weights)

    def run(self):
        with torch.cuda.device(self.device):
            rc = _lib.load().wq_int4_fake_quant_ste_items(self._items.data_ptr(), self.n_items, self.flat_y.data_ptr(),
                                                          self.group, arith.div7_rule(), _lib.stream_ptr(self.device))
        _lib.check(rc, "Int4StePlan.run")
        return self.outputs


class _FakeInt4QuantizationSTEMany(torch.autograd.Function):
    """The same forward for a list of weights in ONE launch (identity backward per weight): the expert weights of a
    grouped linear layer, which the patched forward quantises one after the other (megatron.patch:256-279)."""

    @staticmethod
    def forward(ctx, group_size, *xs):
        device = xs[0].device
        items, n_items, offs, total = _ste_table(xs, group_size)
        flat = torch.empty(total, dtype=torch.bfloat16, device=device)
        with torch.cuda.device(device):
            rc = _lib.load().wq_int4_fake_quant_ste_items(items.data_ptr(), n_items, flat.data_ptr(), int(group_size),
                                                          arith.div7_rule(), _lib.stream_ptr(device))
        _lib.check(rc, "fake_int4_quantization_ste_many")
        return tuple(flat[o:o + x.numel()].view(x.shape) for o, x in zip(offs, xs))

    @staticmethod
    def backward(ctx, *grads):
        return (None,) + tuple(grads)


def fake_int4_quantization_ste_many(xs: Sequence[torch.Tensor], group_size: int):
    """``[fake_int4_quantization_ste(x, group_size) for x in xs]`` with one kernel launch when every weight is a
    contiguous, 16-byte aligned bf16 matrix whose rows are whole groups of 32 / 64 / 128; otherwise one call per
    weight.  Outputs are slices of one fresh allocation."""
    xs = list(xs)
    fast = xs and group_size in (32, 64, 128) and all(
        x.is_cuda and x.dim() == 2 and x.dtype == torch.bfloat16 and x.is_contiguous() and x.data_ptr() % 16 == 0
        and x.numel() and x.shape[1] % group_size == 0 and x.device == xs[0].device for x in xs)
    if not fast:
        return [fake_int4_quantization_ste(x, group_size) for x in xs]
    outs = list(_FakeInt4QuantizationSTEMany.apply(group_size, *xs))
    for x, o in zip(xs, outs):
        if hasattr(x, "main_grad"):
            o.main_grad = x.main_grad
    return outs
