"""ctypes binding of the scalar C oracle (``wq_oracle.c``).  TEST INFRASTRUCTURE ONLY.

Takes and returns CPU torch tensors; all arithmetic happens inside ``libwq_oracle.so``.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libwq_oracle.so")
_lib = None

_i64, _int, _vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "wq_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"], stdout=subprocess.DEVNULL)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        L.wqo_fp8_block_quant.argtypes = [_vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _vp, _vp]
        L.wqo_fp8_block_quant_any.argtypes = [_vp, _int, _i64, _i64, _i64, _i64, _i64, _i64, _int, _vp, _vp]
        L.wqo_fp8_channel_quant.argtypes = [_vp, _i64, _i64, _i64, _i64, _int, _vp, _vp]
        L.wqo_fp8_tensor_quant.argtypes = [_vp, _i64, _i64, _i64, _i64, _int, _vp, _vp]
        L.wqo_fp8_tensor_quant_any.argtypes = [_vp, _int, _i64, _i64, _i64, _i64, _int, _vp, _vp]
        L.wqo_f32_to_f16.argtypes = [ctypes.c_float]
        L.wqo_f32_to_f16.restype = ctypes.c_uint16
        L.wqo_fp8_block_dequant.argtypes = [_vp, _vp, _i64, _i64, _i64, _int, _vp]
        L.wqo_int4_fake_quant.argtypes = [_vp, _int, _i64, _i64, _i64, _i64, _i64, _i64, _int, _vp, _vp, _vp]
        L.wqo_int4_pack_layer.argtypes = [_vp, _i64, _i64, _i64, _int, _vp, _vp, _vp]
        L.wqo_int4_dequant.argtypes = [_vp, _vp, _i64, _i64, _i64, _vp]
        L.wqo_int4_dequant_any.argtypes = [_vp, _vp, _int, _i64, _i64, _i64, _vp]
        L.wqo_int4_fake_ste.argtypes = [_vp, _i64, _i64, _i64, _int, _vp]
        for n in ("wqo_f32_to_e4m3fn_n", "wqo_e4m3fn_to_f32_n", "wqo_f32_to_bf16_n", "wqo_f32_to_f16_n"):
            getattr(L, n).argtypes = [_vp, _vp, _i64]
            getattr(L, n).restype = None
        L.wqo_num_threads.restype = _int
        L.wqo_set_num_threads.argtypes = [_int]
        _lib = L
    return _lib


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what}: oracle rejected the arguments (code {rc})")


def _cpu(t: torch.Tensor) -> torch.Tensor:
    assert t.device.type == "cpu"
    return t


def _cdiv(a, b):
    return -(-a // b)


def f32_to_e4m3fn(x: torch.Tensor) -> torch.Tensor:
    x = _cpu(x).contiguous().to(torch.float32)
    y = torch.empty(x.shape, dtype=torch.uint8)
    lib().wqo_f32_to_e4m3fn_n(x.data_ptr(), y.data_ptr(), x.numel())
    return y


def e4m3fn_to_f32(x: torch.Tensor) -> torch.Tensor:
    x = _cpu(x).contiguous().view(torch.uint8)
    y = torch.empty(x.shape, dtype=torch.float32)
    lib().wqo_e4m3fn_to_f32_n(x.data_ptr(), y.data_ptr(), x.numel())
    return y


def f32_to_bf16(x: torch.Tensor) -> torch.Tensor:
    x = _cpu(x).contiguous().to(torch.float32)
    y = torch.empty(x.shape, dtype=torch.bfloat16)
    lib().wqo_f32_to_bf16_n(x.data_ptr(), y.data_ptr(), x.numel())
    return y


def f32_to_f16(x: torch.Tensor) -> torch.Tensor:
    x = _cpu(x).contiguous().to(torch.float32)
    y = torch.empty(x.shape, dtype=torch.float16)
    lib().wqo_f32_to_f16_n(x.data_ptr(), y.data_ptr(), x.numel())
    return y


def fp8_block_quant(w: torch.Tensor, block_size=(128, 128), mode: int = 0):
    """-> (uint8 [M,N] holding e4m3fn codes, float32 [cdiv(M,bm), cdiv(N,bn)])."""
    assert _cpu(w).dim() == 2
    M, N = w.shape
    bm, bn = int(block_size[0]), int(block_size[1])
    y = torch.empty(M, N, dtype=torch.uint8)
    s = torch.empty(_cdiv(M, bm), _cdiv(N, bn), dtype=torch.float32)
    if w.dtype != torch.bfloat16:
        sel = {torch.float32: 1, torch.float16: 2}[w.dtype]
        _check(lib().wqo_fp8_block_quant_any(w.data_ptr(), sel, M, N, w.stride(0), w.stride(1), bm, bn, mode,
                                             y.data_ptr(), s.data_ptr()), "fp8_block_quant")
        return y, s
    _check(lib().wqo_fp8_block_quant(w.data_ptr(), M, N, w.stride(0), w.stride(1), bm, bn, mode,
                                     y.data_ptr(), s.data_ptr()), "fp8_block_quant")
    return y, s


_ANY_DTYPE = {torch.bfloat16: 0, torch.float32: 1, torch.float16: 2}


def fp8_channel_quant(w: torch.Tensor, mode: int = 0):
    assert _cpu(w).dim() == 2
    if w.dtype != torch.bfloat16:        # a row is a block of shape (1, N): same arithmetic (dimensioned fp32 scale)
        return fp8_block_quant(w, (1, max(w.shape[1], 1)), mode)
    M, N = w.shape
    y = torch.empty(M, N, dtype=torch.uint8)
    s = torch.empty(M, 1, dtype=torch.float32)
    _check(lib().wqo_fp8_channel_quant(w.data_ptr(), M, N, w.stride(0), w.stride(1), mode, y.data_ptr(),
                                       s.data_ptr()),
           "fp8_channel_quant")
    return y, s


def fp8_tensor_quant(w: torch.Tensor, mode: int = 0):
    assert _cpu(w).dim() == 2
    M, N = w.shape
    y = torch.empty(M, N, dtype=torch.uint8)
    s = torch.empty(1, dtype=torch.float32)
    if w.dtype != torch.bfloat16:
        _check(lib().wqo_fp8_tensor_quant_any(w.data_ptr(), _ANY_DTYPE[w.dtype], M, N, w.stride(0), w.stride(1), mode,
                                              y.data_ptr(), s.data_ptr()), "fp8_tensor_quant")
        return y, s
    _check(lib().wqo_fp8_tensor_quant(w.data_ptr(), M, N, w.stride(0), w.stride(1), mode, y.data_ptr(),
                                      s.data_ptr()),
           "fp8_tensor_quant")
    return y, s


def fp8_block_dequant(x: torch.Tensor, s: torch.Tensor, block: int = 128, mode: int = 0) -> torch.Tensor:
    x = _cpu(x).contiguous().view(torch.uint8)
    s = _cpu(s).contiguous().to(torch.float32)
    M, N = x.shape
    assert tuple(s.shape) == (_cdiv(M, block), _cdiv(N, block))
    y = torch.empty(M, N, dtype=torch.bfloat16)
    _check(lib().wqo_fp8_block_dequant(x.data_ptr(), s.data_ptr(), M, N, block, mode, y.data_ptr()),
           "fp8_block_dequant")
    return y


def int4_fake_quant(x: torch.Tensor, block_size, sym: bool):
    assert _cpu(x).dim() == 2 and x.dtype in (torch.bfloat16, torch.float32, torch.float64)
    M, N = x.shape
    bm, bn = int(block_size[0]), int(block_size[1])
    q = torch.empty(M, N, dtype=x.dtype)
    sc = torch.empty(_cdiv(M, bm), _cdiv(N, bn), dtype=x.dtype)
    zp = torch.empty_like(sc)
    sel = {torch.bfloat16: 0, torch.float32: 1, torch.float64: 3}[x.dtype]
    _check(lib().wqo_int4_fake_quant(x.data_ptr(), sel, M, N, x.stride(0),
                                     x.stride(1), bm, bn, int(sym), q.data_ptr(), sc.data_ptr(), zp.data_ptr()),
           "int4_fake_quant")
    return q, sc, zp


def int4_pack_layer(w: torch.Tensor, group_size: int, sym: bool = True):
    w = _cpu(w).contiguous()
    assert w.dtype == torch.bfloat16 and w.dim() == 2
    M, N = w.shape
    packed = torch.empty(M, N // 8, dtype=torch.int32)
    sc = torch.empty(M, N // group_size, dtype=torch.bfloat16)
    pzp = None if sym else torch.empty(N // group_size, M // 8, dtype=torch.int32)
    _check(lib().wqo_int4_pack_layer(w.data_ptr(), M, N, group_size, int(sym), packed.data_ptr(), sc.data_ptr(),
                                     None if sym else pzp.data_ptr()), "int4_pack_layer")
    return packed, sc, pzp


def int4_dequant(packed: torch.Tensor, scale: torch.Tensor, shape, group_size: int) -> torch.Tensor:
    M, N = shape
    packed = _cpu(packed).contiguous()
    scale = _cpu(scale).contiguous()
    assert packed.dtype == torch.int32 and scale.dtype == torch.bfloat16
    y = torch.empty(M, N, dtype=torch.bfloat16)
    _check(lib().wqo_int4_dequant(packed.data_ptr(), scale.data_ptr(), M, N, group_size, y.data_ptr()), "int4_dequant")
    return y


def int4_dequant_any(packed: torch.Tensor, scale: torch.Tensor, shape, group_size: int) -> torch.Tensor:
    """Scale in bf16, fp16 or fp32; group_size <= 0 means one scale per element; N need not be a multiple of 8."""
    M, N = shape
    packed = _cpu(packed).contiguous()
    scale = _cpu(scale).contiguous()
    sel = {torch.bfloat16: 0, torch.float32: 1, torch.float16: 2}[scale.dtype]
    assert packed.dtype == torch.int32 and tuple(packed.shape) == (M, _cdiv(N, 8))
    y = torch.empty(M, N, dtype=torch.bfloat16)
    _check(lib().wqo_int4_dequant_any(packed.data_ptr(), scale.data_ptr(), sel, M, N, group_size if group_size > 0 else 1,
                                      y.data_ptr()), "int4_dequant_any")
    return y


def int4_fake_ste(x: torch.Tensor, group_size: int, div7: int = 0) -> torch.Tensor:
    x = _cpu(x).contiguous()
    assert x.dtype == torch.bfloat16 and x.dim() == 2
    M, N = x.shape
    y = torch.empty(M, N, dtype=torch.bfloat16)
    _check(lib().wqo_int4_fake_ste(x.data_ptr(), M, N, group_size, div7, y.data_ptr()), "int4_fake_ste")
    return y


def num_threads() -> int:
    return lib().wqo_num_threads()
