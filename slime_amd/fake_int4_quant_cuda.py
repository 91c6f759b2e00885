"""Stand-in for the reference's compiled extension module ``fake_int4_quant_cuda``.

Call sites do ``import fake_int4_quant_cuda`` and call ``fake_int4_quant_cuda.fake_int4_quant_cuda(x,
block_size, sym)`` (tools/convert_hf_to_int4_direct.py:26-29,124; quantizer_compressed_tensors.py:236).
Putting this file's directory on ``sys.path`` - or ``sys.modules["fake_int4_quant_cuda"] = this module`` -
routes those calls to the HIP kernel.

Importing this submodule binds the name ``slime_amd.fake_int4_quant_cuda`` to the module, where the package
otherwise exposes the function of the same name; the module is therefore callable and forwards to the function,
so ``slime_amd.fake_int4_quant_cuda(x, block_size, sym)`` keeps working either way.
"""

import sys
import types

from slime_amd.int4 import fake_int4_quant_cuda  # noqa: F401

__all__ = ["fake_int4_quant_cuda"]


class _CallableModule(types.ModuleType):
    def __call__(self, x, block_size, sym):
        return fake_int4_quant_cuda(x, block_size, sym)


sys.modules[__name__].__class__ = _CallableModule
