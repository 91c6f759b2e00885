"""ctypes binding of ``libslime_amd_wq_test.so`` (declared in ``include/slime_amd_wq_test.h``): the on-device self-checks and
the compute-free calibration kernels the tests and the benchmark use.  Not part of the product: nothing under ``slime_amd/``
loads this library."""

from __future__ import annotations

import ctypes
import os
import threading

from slime_amd import _lib

LIB_PATH = os.path.join(os.path.dirname(_lib.LIB_PATH), "libslime_amd_wq_test.so")

_i64, _int, _vp, _u32, _u64 = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint64

SIGNATURES = {
    "wq_test_abi_version": [],
    "wq_selftest_fp8_elem": [_u32, _u32, _int, _vp, _vp],
    "wq_selftest_int4_elem": [_u32, _u32, _vp, _vp],
    "wq_selftest_cvt_fp8": [_u64, _u64, _vp, _vp],
    "wq_selftest_cvt_bf16": [_u64, _u64, _vp, _vp],
    "wq_selftest_decode_fp8": [_vp, _vp],
    "wq_copy_bytes": [_vp, _vp, _i64, _vp],
    "wq_stream_fold_bytes": [_vp, _vp, _i64, _int, _vp],
    "wq_stream_expand_bytes": [_vp, _vp, _i64, _int, _vp],
    "wq_empty_launch": [_i64, _int, _vp],
}

_lib_handle = None
_lock = threading.Lock()


def load() -> ctypes.CDLL:
    global _lib_handle
    with _lock:
        if _lib_handle is None:
            if not os.path.exists(LIB_PATH):
                raise _lib.WqLibraryError(f"{LIB_PATH} not found: build it with `make -C slime_amd/csrc`")
            lib = ctypes.CDLL(LIB_PATH)
            for name, argtypes in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.argtypes, fn.restype = argtypes, _int
            if lib.wq_test_abi_version() != _lib.ABI_VERSION:
                raise _lib.WqLibraryError("libslime_amd_wq_test.so was built against another version of the product header; rebuild")
            _lib_handle = lib
    return _lib_handle
