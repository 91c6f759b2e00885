"""Top-level module ``fake_int4_quant_cuda``: the name of the reference's compiled extension
(slime/backends/megatron_utils/kernels/int4_qat/fake_int4_quant_cuda.cu, built by its setup.py).

The reference's call sites do ``import fake_int4_quant_cuda`` and then
``fake_int4_quant_cuda.fake_int4_quant_cuda(x, block_size, sym)`` (tools/convert_hf_to_int4_direct.py:26-29,124;
megatron_to_hf/processors/quantizer_compressed_tensors.py:236).  With this checkout's root on ``sys.path`` - where the
reference's own extension would be installed - that import resolves here unchanged and runs the gfx950 HIP kernel.
"""

from slime_amd.int4 import fake_int4_quant_cuda  # noqa: F401

__all__ = ["fake_int4_quant_cuda"]
