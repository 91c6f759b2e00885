"""Torch (CPU) restatement of the reference's weight-conversion arithmetic.

TEST INFRASTRUCTURE ONLY.  Nothing in ``slime_amd`` imports this module; it is used by
``tests/``, by the smoke check and by the ``cpu_baseline`` leg of ``bench.py`` as the checker /
the timed CPU path.  Each function applies the same sequence of torch primitives, in the same
dtypes, as the reference function it names, so that on CPU it yields the bytes the reference
yields; the scalar C oracle (``wq_oracle.c``) is the second, independent witness.

Citations are relative to the reference checkout.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F

E4M3 = torch.float8_e4m3fn
E4M3_MAX = torch.finfo(E4M3).max  # 448.0
E4M3_MIN = torch.finfo(E4M3).min  # -448.0


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


# ----------------------------------------------------------------------------- FP8 quant


def _div_scalar(t: torch.Tensor, d: float, device_arith: bool) -> torch.Tensor:
    """``t / d`` for a Python scalar d.  torch evaluates that as a division on CPU tensors and as
    ``t * RN(1/d)`` on GPU tensors; ``device_arith`` reproduces the second form on the CPU."""
    if not device_arith:
        return t / d
    inv = (torch.ones((), dtype=torch.float32) / d).item()
    return t * inv


def block_fp8_ref(w: torch.Tensor, block_size, device_arith: bool = False) -> tuple[torch.Tensor, torch.Tensor]:
    """tools/convert_hf_to_fp8.py:41-75.  pad(0.0) -> view as tiles -> |.|, max over tile rows,
    max over tile cols (weight dtype) -> clamp(min=1e-12) (weight dtype) -> fp32 / 448 ->
    weight / scale (fp32 division) -> clamp(+-448) -> e4m3fn -> crop + contiguous copy."""
    bm, bn = int(block_size[0]), int(block_size[1])
    rows, cols = w.shape
    tm, tn = _cdiv(rows, bm), _cdiv(cols, bn)
    padded = F.pad(w, (0, tn * bn - cols, 0, tm * bm - rows), mode="constant", value=0.0)
    tiles = padded.reshape(tm, bm, tn, bn)
    amax = tiles.abs().max(dim=1, keepdim=True)[0].max(dim=3, keepdim=True)[0]
    scale = _div_scalar(amax.clamp(min=1e-12).to(torch.float32), E4M3_MAX, device_arith)
    q = (tiles / scale).clamp(min=E4M3_MIN, max=E4M3_MAX).reshape(tm * bm, tn * bn).to(E4M3)
    return q[:rows, :cols].clone(), scale.reshape(tm, tn)


def channel_fp8_ref(w: torch.Tensor, device_arith: bool = False) -> tuple[torch.Tensor, torch.Tensor]:
    """tools/convert_hf_to_fp8.py:78-83 (scale shape [M, 1])."""
    amax = w.abs().max(dim=-1, keepdim=True)[0]
    scale = _div_scalar(amax.clamp(min=1e-12).to(torch.float32), E4M3_MAX, device_arith)
    return (w / scale).clamp(min=E4M3_MIN, max=E4M3_MAX).to(E4M3), scale


def tensor_fp8_ref(w: torch.Tensor, device_arith: bool = False) -> tuple[torch.Tensor, torch.Tensor]:
    """tools/convert_hf_to_fp8.py:86-91 and quantizer_fp8.py:114-116 (scale shape [1])."""
    scale = _div_scalar(w.abs().max().clamp(min=1e-12).to(torch.float32), E4M3_MAX, device_arith)
    if device_arith:
        # torch's GPU kernel converts a 0-dim GPU operand to the common dtype (bf16) before dividing
        return (w / scale.to(w.dtype)).clamp(min=E4M3_MIN, max=E4M3_MAX).to(E4M3), scale.view(1)
    return (w / scale).clamp(min=E4M3_MIN, max=E4M3_MAX).to(E4M3), scale.view(1)


def blockwise_cast_ref(x: torch.Tensor, block_size=None, eps: float = 1e-10) -> tuple[torch.Tensor, torch.Tensor]:
    """slime/backends/megatron_utils/kernels/fp8_kernel.py:24-79 read as IEEE fp32 arithmetic:
    per tile, a = max(max|f32(x)|, eps); s = a / 448; y = e4m3(clamp(f32(x) * (1 / s)))."""
    bm, bn = (128, 128) if not block_size else (int(block_size[0]), int(block_size[1]))
    rows, cols = x.shape
    tm, tn = _cdiv(rows, bm), _cdiv(cols, bn)
    x32 = F.pad(x.to(torch.float32), (0, tn * bn - cols, 0, tm * bm - rows), value=0.0).reshape(tm, bm, tn, bn)
    amax = x32.abs().amax(dim=(1, 3), keepdim=True)
    a = torch.maximum(amax, torch.tensor(eps, dtype=torch.float32))
    s = a / torch.tensor(E4M3_MAX, dtype=torch.float32)
    s_inv = torch.tensor(1.0, dtype=torch.float32) / s
    y = (x32 * s_inv).clamp(E4M3_MIN, E4M3_MAX).to(E4M3).reshape(tm * bm, tn * bn)
    return y[:rows, :cols].contiguous(), s.reshape(tm, tn)


# ----------------------------------------------------------------------------- FP8 dequant


def quant_weight_ue8m0_ref(w: torch.Tensor, weight_block_size=(128, 128)) -> tuple[torch.Tensor, torch.Tensor]:
    """The UE8M0 branch of _quantize_param (megatron_to_hf/processors/quantizer_fp8.py:103-106) calls sglang's
    ``quant_weight_ue8m0`` (sglang v0.5.15.post1, not vendored), which applies DeepGEMM's ``per_block_cast_to_fp8`` with
    power-of-two scales.  PARITY UNPINNED: restated from that third-party source as published -
    zero-pad to 128 multiples, ``amax = |x|.float().amax(block).clamp(1e-4)``, ``sf = 2 ** ceil(log2(amax / 448))``,
    ``q = (x * (1 / sf)).to(e4m3fn)`` (no clamp), crop."""
    assert list(weight_block_size) == [128, 128]
    m, n = w.shape
    pm, pn = _cdiv(m, 128) * 128, _cdiv(n, 128) * 128
    padded = torch.zeros((pm, pn), dtype=w.dtype)
    padded[:m, :n] = w
    view = padded.view(-1, 128, pn // 128, 128)
    amax = view.abs().float().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
    sf = amax / 448.0
    sf = torch.pow(2.0, torch.ceil(torch.log2(sf.abs())))
    q = (view * (1.0 / sf)).to(E4M3)
    return q.view_as(padded)[:m, :n].contiguous(), sf.view(view.size(0), view.size(2))


def _expand_scale(s: torch.Tensor, rows: int, cols: int, block: int) -> torch.Tensor:
    return s.repeat_interleave(block, dim=0)[:rows].repeat_interleave(block, dim=1)[:, :cols]


def weight_dequant_ref(x: torch.Tensor, s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """tools/fp8_cast_bf16.py:16-41: y = bf16(f32(x) * s[block]) with one rounding."""
    rows, cols = x.shape
    return (x.to(torch.float32) * _expand_scale(s.to(torch.float32), rows, cols, block_size)).to(torch.bfloat16)


def weight_dequant_bf16_scale_ref(x: torch.Tensor, s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """slime/backends/megatron_utils/hf_to_megatron/common.py:42-56: scale rounded to bf16 first,
    product formed by a bf16 x bf16 multiply."""
    rows, cols = x.shape
    return x.to(torch.bfloat16) * _expand_scale(s.to(torch.bfloat16), rows, cols, block_size)


# ----------------------------------------------------------------------------- INT4


def fake_int4_quant_ref(x: torch.Tensor, block_size, sym: bool):
    """Vectorised restatement of fake_int4_quant_cuda.cu:37-267 for group shapes (bm, bn) that
    tile the reference's 32-lane reduction (bn a multiple of 32 with bm == 1, or bn dividing 32).
    fp32 throughout; outputs cast to x.dtype like the kernel's static_cast stores."""
    bm, bn = int(block_size[0]), int(block_size[1])
    rows, cols = x.shape
    gm, gn = _cdiv(rows, bm), _cdiv(cols, bn)
    x32 = F.pad(x.to(torch.float32), (0, gn * bn - cols, 0, gm * bm - rows), value=0.0).reshape(gm, bm, gn, bn)
    one = torch.tensor(1.0, dtype=torch.float32)
    floor = torch.tensor(1e-5, dtype=torch.float32)
    if sym:
        amax = x32.abs().amax(dim=(1, 3), keepdim=True)
        scale = torch.maximum(amax * (one / 7.0), floor)
        zero = torch.zeros_like(scale)
        q = torch.round(x32 / scale)
    else:
        vmax = x32.amax(dim=(1, 3), keepdim=True)
        vmin = x32.amin(dim=(1, 3), keepdim=True)
        scale = torch.maximum((vmax - vmin) * (one / 15.0), floor)
        zero = (-torch.round(vmin / scale)).clamp(0.0, 15.0) + 0.0  # device fmaxf(-0, +0) is +0
        q = torch.round(x32 / scale) + zero
    q = q.reshape(gm * bm, gn * bn)[:rows, :cols].to(x.dtype).contiguous()
    return q, scale.reshape(gm, gn).to(x.dtype), zero.reshape(gm, gn).to(x.dtype)


def pack_to_int32_ref(value: torch.Tensor, num_bits: int, packed_dim: int = 1, sym: bool = False) -> torch.Tensor:
    """tools/convert_hf_to_int4_direct.py:32-75."""
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
    full = math.ceil(cols / per_word) * per_word
    if full > cols:
        value = F.pad(value, (0, full - cols))
    lanes = value.view(rows, full // per_word, per_word).to(torch.int32)
    shifts = torch.arange(per_word, dtype=torch.int32) * num_bits
    words = (lanes << shifts).sum(dim=2, dtype=torch.int32)
    return words.transpose(0, 1) if packed_dim == 0 else words


def quantize_ref(x: torch.Tensor, scale: torch.Tensor, zero_point, dtype=torch.int8) -> torch.Tensor:
    """tools/convert_hf_to_int4_direct.py:78-120: x / scale (x dtype) [+ zero_point] -> clamp to
    the integer dtype's range -> round half to even -> integer dtype."""
    gs = x.shape[-1] // scale.shape[-1]
    grouped = x.unflatten(-1, (math.ceil(x.shape[-1] / gs), gs))
    scaled = grouped / scale.unsqueeze(-1)
    if zero_point is not None:
        scaled += zero_point.unsqueeze(-1).to(x.dtype)
    info = torch.iinfo(dtype)
    return torch.round(torch.clamp(scaled, info.min, info.max)).to(dtype).flatten(start_dim=-2)


def pack_layer_ref(weight: torch.Tensor, group_size: int, sym: bool = True):
    """tools/convert_hf_to_int4_direct.py:123-153 with the CUDA kernel replaced by
    fake_int4_quant_ref."""
    rows, cols = weight.shape
    q, scale, zp = fake_int4_quant_ref(weight, (1, group_size), sym)
    q = q.view(rows, 1, cols // group_size, group_size)
    scale = scale.view(rows, 1, cols // group_size, 1)
    zp = zp.view(rows, 1, cols // group_size, 1)
    deq = q * scale if sym else (q - zp) * scale
    deq = deq.view(rows, cols)
    scale = scale.view(rows, -1).contiguous()
    if sym:
        zp, packed_zp = None, None
    else:
        zp = zp.view(rows, -1)
        z = zp.t().contiguous().to(torch.float32).to(torch.int32)
        z = z.reshape(-1, z.shape[1] // 8, 8) << (torch.tensor([0, 4, 1, 5, 2, 6, 3, 7]) * 4)
        packed_zp = torch.sum(z, dim=-1).to(torch.int32)
    qi = quantize_ref(deq, scale, zp, torch.int8 if sym else torch.uint8)
    return pack_to_int32_ref(qi, 4, sym=sym), scale, packed_zp


def int4_dequant_ref(packed: torch.Tensor, scale: torch.Tensor, shape, group_size: int) -> torch.Tensor:
    """tools/convert_k2_thinking_int4_to_bf16.py:55-84 with the third-party unpack written out: nibble j of a word
    at bits [4j, 4j+4), minus 8, as int8, rows cut to their length; then the reference's own lines: the scale of any
    dtype ``.to(float32)``, repeated per group (``group_size > 0``) or taken as it is (``group_size <= 0``), reshaped
    to the weight when only the element counts agree, ``(int8.to(f32) * scales).to(bf16)``."""
    rows, cols = shape
    shifts = torch.arange(8, dtype=torch.int32) * 4
    nib = ((packed.unsqueeze(-1) >> shifts) & 0xF).view(rows, -1)[:, :cols]
    q = (nib - 8).to(torch.int8)
    if group_size > 0:
        s = scale.to(torch.float32)
        if s.dim() == 1:
            s = s.unsqueeze(1)
        s = torch.repeat_interleave(s, repeats=group_size, dim=1)
    else:
        s = scale.to(torch.float32)
    if s.shape != q.shape:
        if s.numel() == q.numel():
            s = s.reshape_as(q)
        else:
            raise ValueError(f"Scale shape {s.shape} incompatible with weight shape {q.shape}")
    return (q.to(torch.float32) * s).to(torch.bfloat16).contiguous()


def fake_int4_ste_ref(x: torch.Tensor, group_size: int, device_arith: bool = False) -> torch.Tensor:
    """docker/patch/latest/megatron.patch:212-246 (_FakeInt4QuantizationSTE.forward), op for op."""
    m, n = x.shape
    n_pad = _cdiv(n, group_size) * group_size
    xp = torch.zeros((m, n_pad), dtype=x.dtype, device=x.device)
    xp[:m, :n] = x
    view = xp.view(m, 1, n_pad // group_size, group_size)
    x_max = view.abs().float().amax(dim=(1, 3), keepdim=True)
    x_scale = _div_scalar(x_max, 7, device_arith).clamp(min=1e-5)
    x_q = torch.round(view / x_scale).clamp(-7, 7)
    return (x_q * x_scale).view_as(xp)[:m, :n].contiguous().to(x.dtype)
