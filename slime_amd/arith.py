"""Which of torch's two evaluations of ``tensor / python_scalar`` the torch-formulated functions reproduce.

The reference computes its FP8 scales as ``amax.to(float32) / 448`` (tools/convert_hf_to_fp8.py:65,80,87;
quantizer_fp8.py:114) and the INT4 QAT scale as ``amax / 7`` (docker/patch/latest/megatron.patch:240).  torch
evaluates such an expression as an IEEE division on CPU tensors and as a multiplication by the rounded
reciprocal on GPU tensors; the two differ in the last bit for about half of all amax values.  The reference
runs these functions on the accelerator (convert_hf_to_fp8.py:127) and its test-suite on the CPU
(tests/test_block_fp8_zero_block.py), so both results are "the reference's".

``"device"`` (default): bit-identical to the reference running on a GPU.
``"cpu"``: bit-identical to the reference running on CPU tensors.
The Triton-formulated ``blockwise_cast_to_fp8_triton`` and ``fake_int4_quant_cuda`` are not affected.

The process default comes from ``SLIME_AMD_TORCH_ARITHMETIC`` / ``set_torch_arithmetic``; the ``torch_arithmetic``
context manager overrides it for the calling thread only.
"""

from __future__ import annotations

import contextlib
import contextvars
import os

from . import _lib

_KINDS = ("device", "cpu")
_default = os.environ.get("SLIME_AMD_TORCH_ARITHMETIC", "device")
if _default not in _KINDS:
    raise ValueError(f"SLIME_AMD_TORCH_ARITHMETIC must be one of {_KINDS}, got {_default!r}")

# The setting of the running thread (and of the current asyncio task).  A thread that never chose one sees the
# process default, so `with torch_arithmetic("cpu")` in one worker of a thread pool cannot change what the quantisers
# called from another worker compute.
_local: contextvars.ContextVar = contextvars.ContextVar("slime_amd_torch_arithmetic", default=None)


def _check(kind: str) -> str:
    if kind not in _KINDS:
        raise ValueError(f"torch arithmetic must be one of {_KINDS}, got {kind!r}")
    return kind


def get_torch_arithmetic() -> str:
    return _local.get() or _default


def set_torch_arithmetic(kind: str) -> None:
    """Sets the PROCESS default (what threads without a choice of their own see) and clears this thread's override."""
    global _default
    _default = _check(kind)
    _local.set(None)


@contextlib.contextmanager
def torch_arithmetic(kind: str):
    """Selects the arithmetic for the calling thread (or asyncio task) inside the block; re-entrant; other threads
    are not affected."""
    token = _local.set(_check(kind))
    try:
        yield
    finally:
        _local.reset(token)


def fp8_torch_mode() -> int:
    return _lib.FP8_MODE_TORCH_DEVICE if get_torch_arithmetic() == "device" else _lib.FP8_MODE_TORCH


def div7_rule() -> int:
    return _lib.DIV7_DEVICE if get_torch_arithmetic() == "device" else _lib.DIV7_IEEE
