"""ctypes binding of ``libslime_amd_wq.so`` (the C ABI declared in ``include/slime_amd_wq.h``).

There is no fallback: if the shared library is missing or a symbol cannot be resolved, loading
raises, and every public function of the package raises with it.
"""

from __future__ import annotations

import ctypes
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libslime_amd_wq.so")

ABI_VERSION = 18

# selectors (mirrors of the header's enums)
DTYPE_BF16, DTYPE_F32, DTYPE_F16, DTYPE_F64 = 0, 1, 2, 3
FP8_MODE_TORCH, FP8_MODE_TRITON, FP8_MODE_TORCH_DEVICE, FP8_MODE_UE8M0 = 0, 1, 2, 3
DIV7_IEEE, DIV7_DEVICE = 0, 1
DEQ_MODE_F32SCALE, DEQ_MODE_BF16SCALE = 0, 1
DEQ_SEG, DEQ_SEGS_PER_WG = 512, 16
INT4_GROUPS_PER_WG = 64
INT4_DEQ_WORDS_PER_ITEM = 512
BUCKET_COPY_MARK, BUCKET_COPY_BYTES = -1, 32768
FP8_FEW_MAX = 4

_i64, _int, _vp, _u32, _u64 = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint64

# name -> argtypes; every symbol the header declares is listed here and resolved at load time
SIGNATURES = {
    "wq_abi_version": [],
    "wq_error_string": [_int],
    "wq_fp8_block_quant": [_vp, _i64, _i64, _i64, _i64, _vp, _i64, _vp, _int, _int, _int, _vp],
    "wq_fp8_block_quant_grouped": [_vp, _vp, _int, _i64, _int, _int, _int, _vp],
    "wq_fp8_block_quant_tiles": [_vp, _i64, _int, _int, _int, _vp],
    "wq_fp8_block_quant_few": [_vp, _int, _vp, _int, _int, _int, _vp],
    "wq_fp8_bucket_convert": [_vp, _i64, _vp, _int, _int, _int, _vp],
    "wq_fp8_bucket_convert_rows_off_lines": [_vp, _i64, _vp, _int, _int, _int, _vp],
    "wq_int4_bucket_convert": [_vp, _i64, _vp, _int, _vp],
    "wq_bucket_resolve_items": [_vp, _vp, _vp, _i64, _int, _vp, _vp],
    "wq_fp8_block_quant_any": [_vp, _int, _i64, _i64, _i64, _i64, _vp, _i64, _vp, _int, _int, _int, _vp],
    "wq_fp8_row_quant": [_vp, _i64, _i64, _i64, _i64, _vp, _i64, _vp, _int, _vp],
    "wq_fp8_tensor_quant": [_vp, _i64, _i64, _i64, _i64, _vp, _i64, _vp, _vp, _int, _vp],
    "wq_xxh3_workspace_bytes": [_i64],
    "wq_xxh3_128": [_vp, _i64, _vp, _vp, _vp],
    "wq_xxh3_128_grouped": [_vp, _vp, _int, _i64, _vp],
    "wq_fp8_tensor_quant_any": [_vp, _int, _i64, _i64, _i64, _i64, _vp, _i64, _vp, _vp, _int, _vp],
    "wq_fp8_block_dequant": [_vp, _vp, _vp, _int, _i64, _i64, _int, _int, _vp],
    "wq_fp8_block_quant_dequant": [_vp, _i64, _i64, _i64, _i64, _vp, _i64, _vp, _int, _int, _int, _vp],
    "wq_fp8_block_dequant_grouped": [_vp, _vp, _int, _i64, _int, _int, _int, _vp],
    "wq_fp8_block_dequant_items": [_vp, _i64, _int, _int, _int, _vp],
    "wq_int4_group_quant_pack_asym_items": [_vp, _i64, _vp, _vp, _int, _vp],
    "wq_int4_zero_point_pack_grouped": [_vp, _vp, _int, _i64, _vp, _vp, _vp],
    "wq_int4_fake_quant_ste_items": [_vp, _i64, _vp, _int, _int, _vp],
    "wq_delta_xor_items": [_vp, _i64, _vp, _int, _int, _int, _int, _vp],
    "wq_int4_fake_quant": [_vp, _int, _i64, _i64, _i64, _i64, _int, _int, _int, _vp, _vp, _vp, _vp],
    "wq_int4_group_quant_pack": [_vp, _i64, _i64, _i64, _int, _vp, _vp, _vp],
    "wq_int4_group_quant_pack_grouped": [_vp, _vp, _int, _i64, _int, _vp],
    "wq_int4_group_quant_pack_items": [_vp, _i64, _int, _vp],
    "wq_int4_group_quant_pack_asym": [_vp, _i64, _i64, _i64, _int, _vp, _vp, _vp, _vp],
    "wq_int4_dequant": [_vp, _vp, _vp, _i64, _i64, _int, _vp],
    "wq_int4_dequant_any": [_vp, _vp, _int, _vp, _i64, _i64, _int, _vp],
    "wq_int4_dequant_items": [_vp, _i64, _int, _vp],
    "wq_int4_fake_quant_ste": [_vp, _vp, _i64, _i64, _int, _int, _vp],
    "wq_delta_workspace_bytes": [_i64],
    "wq_delta_xor": [_vp, _vp, _vp, _i64, _int, _vp, _vp, _vp],
    "wq_delta_overwrite_encode": [_vp, _vp, _i64, _vp, ctypes.c_uint32, _vp, _int, _vp],
    "wq_delta_xor_noalloc": [_vp, _vp, _vp, _i64, _int, _vp, _vp],
    "wq_delta_xor_grouped": [_vp, _vp, _int, _i64, _int, _int, _int, _vp],
    "wq_delta_xor_xxh3": [_vp, _vp, _vp, _i64, _int, _vp, _vp, _vp, _vp, _vp],
}

_lib = None
_lock = threading.Lock()


class WqLibraryError(RuntimeError):
    """The HIP library is missing, stale, or a call into it failed."""


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise WqLibraryError(
                f"{LIB_PATH} not found: build it with `make -C slime_amd/csrc` (hipcc, gfx950). "
                "slime_amd has no CPU or pure-torch fallback."
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError as exc:
                raise WqLibraryError(f"{LIB_PATH} does not export {name}; rebuild the library") from exc
            fn.argtypes = argtypes
            fn.restype = (ctypes.c_char_p if name == "wq_error_string"
                          else _i64 if name in ("wq_delta_workspace_bytes", "wq_xxh3_workspace_bytes") else _int)
        if lib.wq_abi_version() != ABI_VERSION:
            raise WqLibraryError(f"ABI mismatch: library {lib.wq_abi_version()}, binding {ABI_VERSION}; rebuild")
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    """RuntimeError on a non-zero return code, like TORCH_CHECK failures of the reference extension."""
    if rc != 0:
        msg = load().wq_error_string(rc).decode()
        raise RuntimeError(f"{what} failed: {msg} (code {rc})")


def stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{what}: input must be on the GPU (got device {t.device}); there is no CPU path")
