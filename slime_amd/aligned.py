"""FP8-aligned training weights: a bf16 weight that holds the values the rollout engine computes with after block-FP8
quantisation, with a straight-through gradient to the trainable weight.

Mirror of ``_get_fp8_aligned_absorb_weight`` / ``_SGLangAbsorbWeightSTE`` (slime_plugins/models/glm5/glm5.py:39-50,
105-165).  The reference quantises (``blockwise_cast_to_fp8_triton`` or sglang's ``quant_weight_ue8m0``) and then
dequantises (sglang's ``block_quant_dequant``) - two kernels, 6 bytes of traffic per element and a code tensor; here one
HIP kernel does both in registers (4 bytes per element) with bit-identical results.
"""

from __future__ import annotations

import torch

from .fp8 import fp8_aligned_weight
from .processors import ue8m0_requant_enabled


class _AbsorbWeightSTE(torch.autograd.Function):
    """Forward: the aligned weight; backward: the gradient goes to the trainable weight unchanged (glm5.py:39-50)."""

    @staticmethod
    def forward(ctx, aligned_weight: torch.Tensor, trainable_weight: torch.Tensor):
        if aligned_weight.shape != trainable_weight.shape:
            raise ValueError(f"Aligned absorb-weight shape mismatch: {aligned_weight.shape} != {trainable_weight.shape}")
        return aligned_weight

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        return None, grad_output


def get_fp8_aligned_absorb_weight(linear: torch.nn.Module, use_ue8m0: bool | None = None) -> torch.Tensor:
    """``linear.weight`` after a 128x128 block-FP8 round trip, recomputed only when the weight changed (the cache key
    is the reference's: version counter, address, device, dtype, shape, strides - plus the scale format) and attached
    to the trainable weight by a straight-through function.  ``use_ue8m0``: power-of-two block scales, as a Blackwell
    rollout dequantises them (glm5.py:128-150); ``None`` follows ``slime_amd.set_ue8m0_requant``."""
    weight = linear.weight
    if use_ue8m0 is None:
        use_ue8m0 = ue8m0_requant_enabled()
    cache_key = (int(weight._version), weight.data_ptr(), weight.device, weight.dtype, tuple(weight.shape),
                 tuple(weight.stride()), bool(use_ue8m0))
    aligned = getattr(linear, "_sglang_fp8_aligned_absorb_weight_cache", None)
    if aligned is None or getattr(linear, "_sglang_fp8_aligned_absorb_weight_cache_key", None) != cache_key:
        with torch.no_grad():
            aligned = fp8_aligned_weight(weight.detach(), (128, 128), use_ue8m0=bool(use_ue8m0))
        linear._sglang_fp8_aligned_absorb_weight_cache = aligned
        linear._sglang_fp8_aligned_absorb_weight_cache_key = cache_key
    return _AbsorbWeightSTE.apply(aligned, weight)
