"""Triton witnesses for the two functions the reference implements as Triton kernels.  TEST INFRASTRUCTURE ONLY
(GPU tests import it; nothing in slime_amd does).

The block-FP8 cast of slime/backends/megatron_utils/kernels/fp8_kernel.py:24-79 and the dequantisation of
tools/fp8_cast_bf16.py:16-41 are defined by what the Triton compiler makes of their arithmetic on the device at
hand - in particular of the two fp32 divisions, which no language rule forces to be IEEE-exact.  These kernels
restate that arithmetic, operation for operation and in the same order (load -> fp32, |x|, max, floor at eps,
divide by 448, reciprocal, multiply, clamp, cast), so that running them on an MI355X shows what the reference
produces there.  The program layout (flat grid, explicit strides) is this file's own.
"""

from __future__ import annotations

import torch
import triton
import triton.language as tl


@triton.jit
def _cast_tile(src, dst, scales, rows, cols, src_rs, src_cs, dst_rs, tiles_per_row, floor_value, lo, hi,
               TM: tl.constexpr, TN: tl.constexpr):
    tile = tl.program_id(0).to(tl.int64)
    ti = tile // tiles_per_row
    tj = tile - ti * tiles_per_row
    r = ti * TM + tl.arange(0, TM)
    c = tj * TN + tl.arange(0, TN)
    inside = (r < rows)[:, None] & (c < cols)[None, :]
    v = tl.load(src + r[:, None] * src_rs + c[None, :] * src_cs, mask=inside, other=0.0).to(tl.float32)
    amax = tl.maximum(tl.max(tl.abs(v)), floor_value)
    scale = amax / hi
    inv = 1.0 / scale
    q = tl.clamp(v * inv, lo, hi).to(dst.dtype.element_ty)
    tl.store(dst + r[:, None] * dst_rs + c[None, :], q, mask=inside)
    tl.store(scales + tile, scale)


def blockwise_cast_triton_ref(x: torch.Tensor, block_size=None, num_warps: int = 8):
    tm, tn = (128, 128) if not block_size else (int(block_size[0]), int(block_size[1]))
    rows, cols = x.shape
    nt_r, nt_c = triton.cdiv(rows, tm), triton.cdiv(cols, tn)
    q = torch.empty(rows, cols, device=x.device, dtype=torch.float8_e4m3fn)
    s = torch.empty(nt_r, nt_c, device=x.device, dtype=torch.float32)
    _cast_tile[(nt_r * nt_c,)](x, q, s, rows, cols, x.stride(0), x.stride(1), q.stride(0), nt_c, 1e-10, -448.0, 448.0,
                               TM=tm, TN=tn, num_warps=num_warps)
    return q, s


@triton.jit
def _dequant_tile(codes, scales, out, rows, cols, tiles_per_row, T: tl.constexpr):
    tile = tl.program_id(0).to(tl.int64)
    ti = tile // tiles_per_row
    tj = tile - ti * tiles_per_row
    r = ti * T + tl.arange(0, T)
    c = tj * T + tl.arange(0, T)
    inside = (r < rows)[:, None] & (c < cols)[None, :]
    at = r[:, None] * cols + c[None, :]
    v = tl.load(codes + at, mask=inside).to(tl.float32)
    sc = tl.load(scales + tile)
    tl.store(out + at, v * sc, mask=inside)


def weight_dequant_triton_ref(x: torch.Tensor, s: torch.Tensor, block_size: int = 128, out_dtype=torch.bfloat16):
    rows, cols = x.shape
    nt_c = triton.cdiv(cols, block_size)
    y = torch.empty(rows, cols, device=x.device, dtype=out_dtype)
    _dequant_tile[(triton.cdiv(rows, block_size) * nt_c,)](x, s, y, rows, cols, nt_c, T=block_size)
    return y
