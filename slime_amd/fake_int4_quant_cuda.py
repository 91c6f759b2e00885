"""Stand-in for the reference's compiled extension module ``fake_int4_quant_cuda``.

Call sites do ``import fake_int4_quant_cuda`` and call ``fake_int4_quant_cuda.fake_int4_quant_cuda(x,
block_size, sym)`` (tools/convert_hf_to_int4_direct.py:26-29,124; quantizer_compressed_tensors.py:236).
Putting this file's directory on ``sys.path`` - or ``sys.modules["fake_int4_quant_cuda"] = this module`` -
routes those calls to the HIP kernel.
"""

from slime_amd.int4 import fake_int4_quant_cuda  # noqa: F401

__all__ = ["fake_int4_quant_cuda"]
