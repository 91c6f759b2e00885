"""slime_amd - MI355X-native low-precision weight conversion for slime.

bf16 -> block-FP8 (e4m3fn, 128x128 blocks, fp32 ``weight_scale_inv``), bf16 -> group-wise INT4
(``weight_packed`` / ``weight_scale`` / ``weight_shape``) and block-FP8 -> bf16, behind the reference's
own function names.  Everything computes in hand-written gfx950 HIP kernels reached through the C ABI
of ``slime_amd/lib/libslime_amd_wq.so``; there is no CPU or pure-torch fallback.
"""

from . import _lib, arith, delta
from .aligned import get_fp8_aligned_absorb_weight
from .hf_reader import SafetensorReader
from .bucket import BucketConverter, FlattenedBucket, FlattenedTensorMetadata, quantize_bucket
from .arith import get_torch_arithmetic, set_torch_arithmetic, torch_arithmetic
from .fp8 import (
    Fp8DequantPlan,
    Fp8QuantPlan,
    block_fp8,
    block_fp8_many,
    block_quant_dequant,
    blockwise_cast_to_fp8_triton,
    channel_fp8,
    fp8_aligned_weight,
    quant_fp8,
    quant_weight_ue8m0,
    tensor_fp8,
    transform_scale_ue8m0,
    weight_dequant,
    weight_dequant_bf16_scale,
)
from .int4 import (
    Int4DequantPlan,
    Int4PackPlan,
    Int4StePlan,
    dequantize_int4,
    fake_int4_quant_cuda,
    fake_int4_quantization_ste,
    fake_int4_quantization_ste_many,
    pack_layer,
    pack_to_int32,
    quantize,
)
from .processors import (
    _quantize_param,
    quantize_params,
    quantize_params_compressed_tensors,
    quantize_grouped_weights,
    quantize_params_fp8,
    set_ue8m0_requant,
)

# the injectable `quantize_weight(weight, (128, 128)) -> (qweight, scale)` hook of the reference's
# alignment forwards (slime/backends/megatron_utils/alignment/deepgemm_moe_forward.py:1145) is this function
quantize_weight = blockwise_cast_to_fp8_triton

__all__ = [
    "quantize_grouped_weights", "block_quant_dequant", "fp8_aligned_weight", "get_fp8_aligned_absorb_weight", "SafetensorReader",
    "Int4StePlan", "fake_int4_quantization_ste_many", "BucketConverter", "FlattenedBucket", "FlattenedTensorMetadata", "quantize_bucket", "quant_weight_ue8m0",
    "set_ue8m0_requant", "transform_scale_ue8m0",
    "Fp8DequantPlan", "Fp8QuantPlan", "Int4DequantPlan", "Int4PackPlan", "block_fp8", "block_fp8_many",
    "blockwise_cast_to_fp8_triton", "channel_fp8", "dequantize_int4", "fake_int4_quant_cuda",
    "fake_int4_quantization_ste", "get_torch_arithmetic", "set_torch_arithmetic", "torch_arithmetic",
    "pack_layer", "pack_to_int32",
    "quant_fp8", "quantize", "quantize_params", "quantize_params_compressed_tensors", "quantize_params_fp8",
    "quantize_weight", "tensor_fp8", "weight_dequant", "weight_dequant_bf16_scale", "_quantize_param",
]
