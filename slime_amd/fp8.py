"""Block-FP8 weight quantisation and dequantisation on MI355X.

Function names, argument meaning, return layouts and error behaviour follow the reference:

* ``block_fp8`` / ``channel_fp8`` / ``tensor_fp8`` / ``quant_fp8``  - tools/convert_hf_to_fp8.py:41-100
* ``blockwise_cast_to_fp8_triton``                                  - slime/backends/megatron_utils/kernels/fp8_kernel.py:61-79
  (the name is kept for call-site compatibility; nothing here uses Triton)
* ``weight_dequant``                                                - tools/fp8_cast_bf16.py:31-41
* ``weight_dequant_bf16_scale``                                     - slime/backends/megatron_utils/hf_to_megatron/common.py:42-56

All arithmetic runs in the HIP kernels of ``libslime_amd_wq.so``.  Inputs live on the GPU; the three torch-formulated
quantisers also take host tensors, as the reference's do, by way of the GPU (see ``_host_tensor_through_gpu``).
``Fp8QuantPlan`` / ``Fp8DequantPlan`` quantise many tensors with ONE kernel launch and write into
one flat output buffer - the shape a weight-sync bucket wants.
"""

from __future__ import annotations

from typing import Sequence

import torch

from . import _lib, arith

FP8_DTYPE = torch.float8_e4m3fn
FP8_INFO = torch.finfo(FP8_DTYPE)
FP8_MAX, FP8_MIN = FP8_INFO.max, FP8_INFO.min


def ceildiv(a: int, b: int) -> int:
    return -(-a // b)


def _check_weight(w: torch.Tensor, what: str) -> None:
    _lib.require_gpu(w, what)
    if w.dim() != 2:
        raise ValueError(f"{what}: expected a 2-D weight, got shape {tuple(w.shape)}")
    if w.dtype != torch.bfloat16:
        raise TypeError(f"{what}: only bfloat16 weights are supported (got {w.dtype})")


_OTHER_FLOAT_DTYPES = {torch.float16: _lib.DTYPE_F16, torch.float32: _lib.DTYPE_F32}


def _host_tensor_through_gpu(fn, weight: torch.Tensor, what: str, *args):
    """The reference's ``block_fp8`` / ``channel_fp8`` / ``tensor_fp8`` are plain torch ops and take host tensors (its own
    test, tests/test_block_fp8_zero_block.py, runs them on the CPU).  A host tensor is uploaded, quantised by the same
    kernels in the arithmetic torch uses on CPU tensors - which is what the reference computes for such an input - and the
    results are handed back on the host.  No GPU: RuntimeError, as for every entry point of the package."""
    if not torch.cuda.is_available():
        _lib.require_gpu(weight, what)
    device = torch.device("cuda", torch.cuda.current_device())
    with arith.torch_arithmetic("cpu"):
        q, s = fn(weight.to(device), *args)
    return q.cpu(), s.cpu()


def _block_quant(w: torch.Tensor, bm: int, bn: int, mode: int, what: str):
    """bf16 weights take the bandwidth-tuned kernel; fp16 / fp32 weights, which the reference functions also accept,
    a plain one with the reference's arithmetic for that dtype."""
    if w.dtype in _OTHER_FLOAT_DTYPES:
        _lib.require_gpu(w, what)
        if w.dim() != 2:
            raise ValueError(f"{what}: expected a 2-D weight, got shape {tuple(w.shape)}")
    else:
        _check_weight(w, what)
    if bm <= 0 or bn <= 0:
        raise ValueError(f"{what}: block size must be positive, got {(bm, bn)}")
    M, N = w.shape
    q = torch.empty((M, N), dtype=FP8_DTYPE, device=w.device)
    s = torch.empty((ceildiv(M, bm), ceildiv(N, bn)), dtype=torch.float32, device=w.device)
    if M and N:
        with torch.cuda.device(w.device):
            if w.dtype == torch.bfloat16:
                rc = _lib.load().wq_fp8_block_quant(w.data_ptr(), M, N, w.stride(0), w.stride(1), q.data_ptr(), N,
                                                    s.data_ptr(), bm, bn, mode, _lib.stream_ptr(w.device))
            else:
                rc = _lib.load().wq_fp8_block_quant_any(w.data_ptr(), _OTHER_FLOAT_DTYPES[w.dtype], M, N, w.stride(0),
                                                        w.stride(1), q.data_ptr(), N, s.data_ptr(), bm, bn, mode,
                                                        _lib.stream_ptr(w.device))
        _lib.check(rc, what)
    return q, s


def block_fp8(weight: torch.Tensor, block_size) -> tuple[torch.Tensor, torch.Tensor]:
    """-> (qweight float8_e4m3fn [M,N] contiguous, scale float32 [ceil(M/bn), ceil(N/bk)]).

    Arithmetic of tools/convert_hf_to_fp8.py:41-75: zero padding of edge blocks, amax clamped at
    1e-12 in the weight dtype, scale = f32(amax)/448, q = clamp(f32(w)/scale), RNE to e4m3fn.  `/448` is
    evaluated as torch does on GPU tensors unless ``arith.set_torch_arithmetic("cpu")`` is in force.  A host tensor is
    quantised on the GPU in the CPU evaluation and comes back on the host."""
    if isinstance(weight, torch.Tensor) and not weight.is_cuda:
        return _host_tensor_through_gpu(block_fp8, weight, "block_fp8", block_size)
    return _block_quant(weight, int(block_size[0]), int(block_size[1]), arith.fp8_torch_mode(), "block_fp8")


def channel_fp8(weight: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-row scaling, tools/convert_hf_to_fp8.py:78-83 -> (qweight [M,N], scale float32 [M,1]).  bf16 rows take the
    bandwidth-tuned kernels; fp16 / fp32 weights are quantised as blocks of one row (the same arithmetic: both
    divide by a dimensioned float32 scale)."""
    if isinstance(weight, torch.Tensor) and not weight.is_cuda:
        return _host_tensor_through_gpu(channel_fp8, weight, "channel_fp8")
    if weight.dtype in _OTHER_FLOAT_DTYPES and weight.dim() == 2:
        return _block_quant(weight, 1, max(int(weight.shape[1]), 1), arith.fp8_torch_mode(), "channel_fp8")
    _check_weight(weight, "channel_fp8")
    M, N = weight.shape
    q = torch.empty((M, N), dtype=FP8_DTYPE, device=weight.device)
    s = torch.empty((M, 1), dtype=torch.float32, device=weight.device)
    if M:
        with torch.cuda.device(weight.device):
            rc = _lib.load().wq_fp8_row_quant(weight.data_ptr(), M, N, weight.stride(0), weight.stride(1),
                                              q.data_ptr(), N, s.data_ptr(), arith.fp8_torch_mode(),
                                              _lib.stream_ptr(weight.device))
        _lib.check(rc, "channel_fp8")
    return q, s


def tensor_fp8(weight: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-tensor scaling, tools/convert_hf_to_fp8.py:86-91 -> (qweight [M,N], scale float32 [1]).  The quotient is
    rounded to the weight's dtype before the clamp, as torch's type promotion with a 0-dim scale makes it (bf16 and
    fp16 weights round twice, fp32 weights once); fp16 / fp32 weights take plain two-pass kernels."""
    if isinstance(weight, torch.Tensor) and not weight.is_cuda:
        return _host_tensor_through_gpu(tensor_fp8, weight, "tensor_fp8")
    other = weight.dtype in _OTHER_FLOAT_DTYPES and weight.dim() == 2
    if other:
        _lib.require_gpu(weight, "tensor_fp8")
    else:
        _check_weight(weight, "tensor_fp8")
    M, N = weight.shape
    q = torch.empty((M, N), dtype=FP8_DTYPE, device=weight.device)
    s = torch.empty((1,), dtype=torch.float32, device=weight.device)
    ws = torch.zeros((1,), dtype=torch.int32, device=weight.device)
    with torch.cuda.device(weight.device):
        if other:
            rc = _lib.load().wq_fp8_tensor_quant_any(weight.data_ptr(), _OTHER_FLOAT_DTYPES[weight.dtype], M, N,
                                                     weight.stride(0), weight.stride(1), q.data_ptr(), N, s.data_ptr(),
                                                     ws.data_ptr(), arith.fp8_torch_mode(), _lib.stream_ptr(weight.device))
        else:
            rc = _lib.load().wq_fp8_tensor_quant(weight.data_ptr(), M, N, weight.stride(0), weight.stride(1),
                                                 q.data_ptr(), N, s.data_ptr(), ws.data_ptr(), arith.fp8_torch_mode(),
                                                 _lib.stream_ptr(weight.device))
    _lib.check(rc, "tensor_fp8")
    return q, s


def quant_fp8(weight: torch.Tensor, strategy: str, block_size=None):
    """Dispatcher of tools/convert_hf_to_fp8.py:94-100 ("tensor", "channel", anything else = block)."""
    if strategy == "tensor":
        return tensor_fp8(weight)
    if strategy == "channel":
        return channel_fp8(weight)
    return block_fp8(weight, block_size)


def blockwise_cast_to_fp8_triton(x: torch.Tensor, block_size=None) -> tuple[torch.Tensor, torch.Tensor]:
    """Weight-sync variant (fp8_kernel.py:61-79): fp32 amax floored at 1e-10, y = x * (1/scale).
    Accepts any strides, like the kernel it replaces; block size defaults to 128x128."""
    bm, bn = (128, 128) if not block_size else (int(block_size[0]), int(block_size[1]))
    return _block_quant(x, bm, bn, _lib.FP8_MODE_TRITON, "blockwise_cast_to_fp8_triton")


def quant_weight_ue8m0(weight_dequant: torch.Tensor, weight_block_size) -> tuple[torch.Tensor, torch.Tensor]:
    """Block quantisation with power-of-two (UE8M0) scales: the function the reference imports from sglang and calls
    at quantizer_fp8.py:103-106 when the rollout engine wants DeepGEMM's scale format.  -> (qweight e4m3fn [M,N],
    scale float32 [ceil(M/128), ceil(N/128)], every entry a power of two).  The arithmetic - fp32 amax floored at
    1e-4, ``sf = 2 ** ceil(log2(amax / 448))``, ``q = x * (1 / sf)`` - is restated from sglang / DeepGEMM, which the
    reference does not vendor: bit parity with them is unpinned.  bf16 weights, 128x128 blocks."""
    assert list(weight_block_size) == [128, 128]
    if weight_dequant.dtype != torch.bfloat16:
        raise TypeError(f"quant_weight_ue8m0: only bfloat16 weights are supported (got {weight_dequant.dtype})")
    n, k = weight_dequant.shape[-2:]
    q, s = _block_quant(weight_dequant.reshape(-1, k), 128, 128, _lib.FP8_MODE_UE8M0, "quant_weight_ue8m0")
    lead = tuple(weight_dequant.shape[:-2])
    if lead:
        if n % 128:
            raise ValueError("quant_weight_ue8m0: batched weights need a row count that is a multiple of 128")
        return q.view(weight_dequant.shape), s.view(*lead, n // 128, ceildiv(k, 128))
    return q, s


def transform_scale_ue8m0(sf: torch.Tensor, mn: int) -> torch.Tensor:
    """Not provided.  The reference's ``transform_scale_ue8m0`` (sglang) repacks the scales into DeepGEMM's MN-major,
    TMA-aligned, four-exponents-per-int32 layout - a memory layout of NVIDIA's tensor memory accelerator that no kernel
    on this hardware reads, defined by a library the reference does not vendor."""
    raise NotImplementedError(
        "transform_scale_ue8m0: DeepGEMM's packed TMA-aligned UE8M0 layout is NVIDIA-specific and is not produced here; "
        "call with transform_ue8m0=False to get the power-of-two scales as float32 (the form hf_checkpoint_saver uses)")


_DEQ_OUT_DTYPES = {torch.bfloat16: _lib.DTYPE_BF16, torch.float32: _lib.DTYPE_F32, torch.float16: _lib.DTYPE_F16}


def _dequant(x: torch.Tensor, s: torch.Tensor, block_size: int, mode: int, out_dtype: torch.dtype, what: str):
    _lib.require_gpu(x, what)
    assert x.is_contiguous() and s.is_contiguous()
    assert x.dim() == 2 and s.dim() == 2
    if x.element_size() != 1:
        raise TypeError(f"{what}: x must hold one-byte e4m3fn codes, got {x.dtype}")
    if s.dtype != torch.float32:
        raise TypeError(f"{what}: scale must be float32, got {s.dtype}")
    if out_dtype not in _DEQ_OUT_DTYPES or (out_dtype == torch.float16 and mode != _lib.DEQ_MODE_F32SCALE):
        raise TypeError(f"{what}: output dtype {out_dtype} is not supported (bfloat16, float16 or float32)")
    M, N = x.shape
    if tuple(s.shape) != (ceildiv(M, block_size), ceildiv(N, block_size)):
        raise ValueError(f"{what}: scale shape {tuple(s.shape)} does not match x {tuple(x.shape)} / {block_size}")
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    if M and N:
        with torch.cuda.device(x.device):
            rc = _lib.load().wq_fp8_block_dequant(
                x.data_ptr(), s.data_ptr(), y.data_ptr(),
                _DEQ_OUT_DTYPES[out_dtype], M, N, int(block_size), mode, _lib.stream_ptr(x.device))
        _lib.check(rc, what)
    return y


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """y = (f32(x) * s[block]) in torch's default dtype (tools/fp8_cast_bf16.py:31-41; the tool sets the
    default dtype to bfloat16 at :45, callers that have not get float32 - or float16 -, as with the reference)."""
    return _dequant(x, s, block_size, _lib.DEQ_MODE_F32SCALE, torch.get_default_dtype(), "weight_dequant")


def block_quant_dequant(x_q_block: torch.Tensor, x_s: torch.Tensor, block_size, dtype: torch.dtype) -> torch.Tensor:
    """Name and arguments of the sglang helper the reference calls at slime_plugins/models/glm5/glm5.py:144-161
    (``block_quant_dequant(qweight, scale_inv, [128, 128], torch.bfloat16)``): e4m3fn codes times their block scale in
    fp32, rounded once to ``dtype`` (bfloat16 or float32) - ``weight_dequant``'s arithmetic with an explicit output
    type.  Square blocks only (the dequantiser's contract)."""
    bm, bn = int(block_size[0]), int(block_size[1])
    if bm != bn:
        raise ValueError(f"block_quant_dequant: square blocks only, got {bm}x{bn}")
    return _dequant(x_q_block, x_s, bm, _lib.DEQ_MODE_F32SCALE, dtype, "block_quant_dequant")


def fp8_aligned_weight(weight: torch.Tensor, block_size=(128, 128), use_ue8m0: bool = False,
                       return_scale: bool = False):
    """bf16 weight -> bf16 weight holding the values it has after block-FP8 quantisation, in ONE pass (2 + 2 bytes per
    element instead of 3 + 3 and no code tensor).  Bit-identical to the pair the reference runs in
    ``_get_fp8_aligned_absorb_weight`` (slime_plugins/models/glm5/glm5.py:105-165)::

        block_quant_dequant(*blockwise_cast_to_fp8_triton(w.contiguous(), (128, 128)), [128, 128], torch.bfloat16)
        block_quant_dequant(*quant_weight_ue8m0(w.contiguous(), [128, 128]), [128, 128], torch.bfloat16)   # use_ue8m0

    Any row / column strides; ``return_scale`` also returns the float32 block scales."""
    _check_weight(weight, "fp8_aligned_weight")
    bm, bn = int(block_size[0]), int(block_size[1])
    if bm <= 0 or bn <= 0:
        raise ValueError(f"fp8_aligned_weight: block size must be positive, got {block_size}")
    M, N = weight.shape
    y = torch.empty((M, N), dtype=torch.bfloat16, device=weight.device)
    s = torch.empty((ceildiv(M, bm), ceildiv(N, bn)), dtype=torch.float32, device=weight.device) if return_scale else None
    if M and N:
        with torch.cuda.device(weight.device):
            rc = _lib.load().wq_fp8_block_quant_dequant(
                weight.data_ptr(), M, N, weight.stride(0), weight.stride(1), y.data_ptr(), N,
                s.data_ptr() if return_scale else None, bm, bn,
                _lib.FP8_MODE_UE8M0 if use_ue8m0 else _lib.FP8_MODE_TRITON, _lib.stream_ptr(weight.device))
        _lib.check(rc, "fp8_aligned_weight")
    return (y, s) if return_scale else y


def weight_dequant_bf16_scale(x: torch.Tensor, s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """Dequant-on-read of the HF->Megatron loader (hf_to_megatron/common.py:42-56): the scale is
    rounded to bf16 before the multiply; result bf16."""
    return _dequant(x, s, block_size, _lib.DEQ_MODE_BF16SCALE, torch.bfloat16, "weight_dequant_bf16_scale")


# ------------------------------------------------------------------------------------ grouped launches


def _align(n: int, a: int = 256) -> int:
    return (n + a - 1) // a * a


_ITEM_TABLE_MIN_TENSORS = 64     # plans with at least this many tensors pre-resolve every work item on the host


def _to_device_i64(rows, device) -> torch.Tensor:
    return torch.tensor(rows, dtype=torch.int64).to(device)


def tile_table(rows, bm: int, bn: int):
    """One descriptor per (bm x bn) tile, moved to the tile's origin, from per-tensor rows
    ``[x, y, s, M, N, sx_m, sx_n, sy_m]`` (addresses, or byte offsets for the bucket launches; sizes and strides in
    elements).  -> (int64 [tiles, 8] in tensor order, row-major tiles within a tensor; owner index per tile)."""
    desc = torch.as_tensor(rows, dtype=torch.int64).reshape(-1, 8)
    tm, tn = (desc[:, 3] + bm - 1) // bm, (desc[:, 4] + bn - 1) // bn
    counts = tm * tn
    owner = torch.repeat_interleave(torch.arange(desc.shape[0]), counts)
    local = torch.arange(int(counts.sum()), dtype=torch.int64) - (torch.cumsum(counts, 0) - counts)[owner]
    d = desc[owner]
    kt = tn[owner]
    r0, c0 = (local // kt) * bm, (local % kt) * bn
    table = torch.stack([d[:, 0] + (r0 * d[:, 5] + c0 * d[:, 6]) * 2, d[:, 1] + r0 * d[:, 7] + c0,
                         d[:, 2] + local * 4, d[:, 3] - r0, d[:, 4] - c0, d[:, 5], d[:, 6], d[:, 7]], dim=1)
    return table, owner, local


class Fp8QuantPlan:
    """Quantise a fixed list of bf16 weights with one kernel launch per ``run()``.

    Outputs live in two flat buffers owned by the plan (``flat_q`` bytes, ``flat_s`` fp32); ``outputs``
    holds per-tensor views ``(qweight [M,N] e4m3fn, scale [tm,tn])`` in input order.  The plan reads
    the weights' current contents on every run, so it can be reused across weight-sync steps as long
    as the input tensors stay at the same addresses.  mode: None = ``block_fp8`` arithmetic under the
    current ``arith`` setting, 0 / 2 = ``block_fp8`` as torch evaluates it on CPU / GPU tensors,
    1 = ``blockwise_cast_to_fp8_triton`` arithmetic.
    """

    def __init__(self, weights: Sequence[torch.Tensor], block_size=(128, 128), mode: int | None = None):
        if not weights:
            raise ValueError("Fp8QuantPlan: empty weight list")
        self.bm, self.bn = int(block_size[0]), int(block_size[1])
        self.mode = arith.fp8_torch_mode() if mode is None else int(mode)
        self.device = weights[0].device
        self.weights = list(weights)
        q_off, s_off, q_total, s_total = [], [], 0, 0
        for w in self.weights:
            _check_weight(w, "Fp8QuantPlan")
            if w.device != self.device:
                raise ValueError("Fp8QuantPlan: all weights must be on one device")
            M, N = w.shape
            q_off.append(q_total)
            s_off.append(s_total)
            q_total += _align(M * N)
            s_total += _align(ceildiv(M, self.bm) * ceildiv(N, self.bn) * 4) // 4
        self.flat_q = torch.empty(max(q_total, 1), dtype=torch.uint8, device=self.device)
        self.flat_s = torch.empty(max(s_total, 1), dtype=torch.float32, device=self.device)
        rows, starts, tiles = [], [0], 0
        self.outputs = []
        for w, qo, so in zip(self.weights, q_off, s_off):
            M, N = w.shape
            tm, tn = ceildiv(M, self.bm), ceildiv(N, self.bn)
            q = self.flat_q[qo:qo + M * N].view(FP8_DTYPE).view(M, N)
            s = self.flat_s[so:so + tm * tn].view(tm, tn)
            self.outputs.append((q, s))
            rows.append([w.data_ptr(), q.data_ptr(), s.data_ptr(), M, N, w.stride(0), w.stride(1), N])
            tiles += tm * tn
            starts.append(tiles)
        self.total_tiles = tiles
        self.bf16_bytes = sum(2 * w.numel() for w in self.weights)
        # Many small tensors: one descriptor per tile, moved to the tile's origin (64 bytes per 48 KiB of traffic), so
        # that the kernel needs a single scalar load instead of a search through the per-tensor prefix sums.  A
        # handful of tensors (the q/k/v or gate/up group of one weight-sync call) keeps the search: it is short
        # there and the table would cost more host time to build than it saves.
        self._tiles = None
        if len(rows) >= _ITEM_TABLE_MIN_TENSORS:
            table, _, _ = tile_table(rows, self.bm, self.bn)             # rows: x, y, s, M, N, sx_m, sx_n, sy_m
            self._tiles = table.contiguous().to(self.device)
        else:
            self._descs = _to_device_i64(rows, self.device)
            self._starts = _to_device_i64(starts, self.device)

    def run(self):
        lib = _lib.load()
        with torch.cuda.device(self.device):
            if self._tiles is not None:
                rc = lib.wq_fp8_block_quant_tiles(self._tiles.data_ptr(), self.total_tiles, self.bm, self.bn, self.mode,
                                                  _lib.stream_ptr(self.device))
            else:
                rc = lib.wq_fp8_block_quant_grouped(self._descs.data_ptr(), self._starts.data_ptr(), len(self.weights),
                                                    self.total_tiles, self.bm, self.bn, self.mode,
                                                    _lib.stream_ptr(self.device))
        _lib.check(rc, "Fp8QuantPlan.run")
        return self.outputs


def block_fp8_many(weights: Sequence[torch.Tensor], block_size=(128, 128), mode: int | None = None):
    """One-launch ``block_fp8`` over a list of weights -> list of (qweight, scale)."""
    return Fp8QuantPlan(weights, block_size, mode).run() if weights else []


class Fp8DequantPlan:
    """One-launch block-FP8 -> bf16 over a fixed list of (codes, scale_inv) pairs; see Fp8QuantPlan."""

    def __init__(self, xs: Sequence[torch.Tensor], ss: Sequence[torch.Tensor], block_size: int = 128,
                 mode: int = 0, out_dtype: torch.dtype = torch.bfloat16):
        if not xs or len(xs) != len(ss):
            raise ValueError("Fp8DequantPlan: need equally many code and scale tensors")
        if out_dtype not in (torch.bfloat16, torch.float32):
            raise TypeError(f"Fp8DequantPlan: output dtype {out_dtype} is not supported")
        self.block, self.mode, self.out_dtype = int(block_size), int(mode), out_dtype
        self.device = xs[0].device
        self.xs, self.ss = list(xs), list(ss)
        esz = 2 if out_dtype == torch.bfloat16 else 4
        offs, total = [], 0
        for x, s in zip(self.xs, self.ss):
            _lib.require_gpu(x, "Fp8DequantPlan")
            assert x.is_contiguous() and s.is_contiguous() and x.dim() == 2 and s.dim() == 2
            assert x.element_size() == 1 and s.dtype == torch.float32
            M, N = x.shape
            assert tuple(s.shape) == (ceildiv(M, self.block), ceildiv(N, self.block))
            if N >= 2 ** 31 or M * ceildiv(N, _lib.DEQ_SEG) >= 2 ** 31:
                raise ValueError("Fp8DequantPlan: tensor too large for one descriptor; split it by rows")
            offs.append(total)
            total += _align(M * N * esz) // esz
        self.flat_y = torch.empty(max(total, 1), dtype=out_dtype, device=self.device)
        rows, starts, work = [], [0], 0
        self.outputs = []
        for x, s, o in zip(self.xs, self.ss, offs):
            M, N = x.shape
            y = self.flat_y[o:o + M * N].view(M, N)
            self.outputs.append(y)
            rows.append([x.data_ptr(), s.data_ptr(), y.data_ptr(), M, N])
            work += ceildiv(M * ceildiv(N, _lib.DEQ_SEG), _lib.DEQ_SEGS_PER_WG)
            starts.append(work)
        self.total_work = work
        self.out_bytes = sum(x.numel() * esz for x in self.xs)
        # many tensors: one pre-resolved descriptor per work item (48 bytes per 24 KiB of traffic) instead of the search
        self._items = None
        if len(rows) >= _ITEM_TABLE_MIN_TENSORS:
            desc = torch.tensor(rows, dtype=torch.int64)
            start = torch.tensor(starts, dtype=torch.int64)
            owner = torch.repeat_interleave(torch.arange(len(rows)), start[1:] - start[:-1])
            local = torch.arange(work, dtype=torch.int64) - start[owner]
            self._items = torch.cat([desc[owner], local.unsqueeze(1)], dim=1).contiguous().to(self.device)
        else:
            self._descs = _to_device_i64(rows, self.device)
            self._starts = _to_device_i64(starts, self.device)

    def run(self):
        out_sel = _lib.DTYPE_BF16 if self.out_dtype == torch.bfloat16 else _lib.DTYPE_F32
        with torch.cuda.device(self.device):
            if self._items is not None:
                rc = _lib.load().wq_fp8_block_dequant_items(self._items.data_ptr(), self.total_work, out_sel, self.block,
                                                            self.mode, _lib.stream_ptr(self.device))
            else:
                rc = _lib.load().wq_fp8_block_dequant_grouped(
                    self._descs.data_ptr(), self._starts.data_ptr(), len(self.xs), self.total_work, out_sel,
                    self.block, self.mode, _lib.stream_ptr(self.device))
        _lib.check(rc, "Fp8DequantPlan.run")
        return self.outputs
