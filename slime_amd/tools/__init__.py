"""Offline checkpoint converters with the command lines and on-disk formats of the reference's tools/:

* ``python -m slime_amd.tools.convert_hf_to_fp8``         - tools/convert_hf_to_fp8.py
* ``python -m slime_amd.tools.fp8_cast_bf16``             - tools/fp8_cast_bf16.py
* ``python -m slime_amd.tools.convert_hf_to_int4_direct`` - tools/convert_hf_to_int4_direct.py

Every shard is converted with one grouped kernel launch on the GPU.
"""
