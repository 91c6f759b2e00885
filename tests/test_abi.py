"""The C-ABI library loads without a GPU, exports every symbol the header declares, and rejects bad
arguments before launching anything (no compute calls here)."""

import ctypes
import os
import re

import pytest

import wq_testlib
from slime_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "slime_amd_wq.h")
TEST_HEADER = os.path.join(ROOT, "include", "slime_amd_wq_test.h")


def _declared_symbols(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(wq_[a-z0-9_]+)\s*\(", text)))


def _exported_symbols(path):
    import subprocess

    out = subprocess.check_output(["nm", "-D", "--defined-only", path], text=True)
    return sorted(ln.split()[-1] for ln in out.splitlines() if " T " in ln and ln.split()[-1].startswith("wq_"))


def test_header_symbols_are_exported_and_bound():
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 15
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names
    assert _exported_symbols(_lib.LIB_PATH) == names        # nothing exported that the header does not declare


def test_product_library_holds_no_instruments():
    """Self-checks and calibration kernels live in a library of their own: the product header declares only entry points
    that replace a reference interface (plus the no-allocation variant), and the two libraries share no symbol."""
    product, instruments = _declared_symbols(), _declared_symbols(TEST_HEADER)
    assert not [n for n in product if "selftest" in n or n in ("wq_copy_bytes", "wq_stream_fold_bytes", "wq_empty_launch")]
    assert not set(product) & set(instruments)
    assert sorted(wq_testlib.SIGNATURES) == instruments == _exported_symbols(wq_testlib.LIB_PATH)
    lib = wq_testlib.load()
    assert lib.wq_test_abi_version() == _lib.ABI_VERSION


def test_abi_version_and_error_strings():
    lib = _lib.load()
    assert lib.wq_abi_version() == _lib.ABI_VERSION
    for code in (0, -1, -2, -3, -4, -5, -6):
        assert lib.wq_error_string(code)
    assert lib.wq_error_string(-99) == b"unknown error"


def test_argument_validation_without_launch():
    lib = _lib.load()
    S, M_, U, N_ = -2, -3, -4, -1
    assert lib.wq_fp8_block_quant(None, -1, 4, 4, 1, None, 4, None, 128, 128, 0, None) == S
    assert lib.wq_fp8_block_quant(None, 4, 4, 4, 1, None, 4, None, 0, 128, 0, None) == S
    assert lib.wq_fp8_block_quant(None, 4, 4, 4, 1, None, 4, None, 128, 128, 7, None) == M_
    assert lib.wq_fp8_block_quant(None, 4, 4, 4, 1, None, 4, None, 128, 128, 0, None) == N_
    assert lib.wq_fp8_block_quant(None, 0, 4, 4, 1, None, 4, None, 128, 128, 0, None) == 0      # empty: no-op
    assert lib.wq_fp8_block_quant_grouped(None, None, 3, 10, 128, 128, 0, None) == N_
    assert lib.wq_fp8_block_quant_grouped(None, None, 0, 0, 128, 128, 0, None) == 0
    assert lib.wq_fp8_block_quant_tiles(None, 4, 128, 128, 0, None) == N_
    assert lib.wq_fp8_block_quant_tiles(None, 4, 128, 128, 9, None) == M_
    assert lib.wq_fp8_block_quant_tiles(None, 0, 128, 128, 0, None) == 0
    assert lib.wq_fp8_block_quant(None, 4, 4, 4, 1, None, 4, None, 128, 128, 2, None) == N_
    assert lib.wq_fp8_block_quant_few(None, 5, None, 128, 128, 1, None) == S           # more than WQ_FP8_FEW_MAX
    assert lib.wq_fp8_block_quant_few(None, 2, None, 128, 128, 1, None) == N_
    assert lib.wq_fp8_block_quant_few(None, 0, None, 128, 128, 1, None) == 0
    assert lib.wq_bucket_resolve_items(None, None, None, 3, 8, None, None) == N_
    assert lib.wq_bucket_resolve_items(None, None, None, 3, 0, None, None) == S
    assert lib.wq_bucket_resolve_items(ctypes.c_void_p(64), ctypes.c_void_p(64), ctypes.c_void_p(64), 3, 8, ctypes.c_void_p(64), None) == U
    assert lib.wq_fp8_row_quant(None, -1, 4, 4, 1, None, 4, None, 0, None) == S
    assert lib.wq_fp8_row_quant(None, 4, 4, 4, 1, None, 4, None, 1, None) == M_         # no Triton row form
    assert lib.wq_fp8_tensor_quant(None, 4, 4, 4, 1, None, 4, None, None, 2, None) == N_
    assert lib.wq_fp8_tensor_quant(None, 4, 4, 4, 1, None, 4, None, None, 1, None) == M_
    assert lib.wq_fp8_block_dequant(None, None, None, 0, 4, 4, 0, 0, None) == S
    assert lib.wq_fp8_block_dequant(None, None, None, 5, 4, 4, 128, 0, None) == M_
    assert lib.wq_fp8_block_dequant(None, None, None, 0, 4, 4, 128, 0, None) == N_
    assert lib.wq_fp8_block_dequant_grouped(None, None, 1, 1, 0, 128, 3, None) == M_
    assert lib.wq_int4_fake_quant(None, 0, 4, 64, 64, 1, 1, 48, 1, None, None, None, None) == S
    assert lib.wq_int4_fake_quant(None, 0, 4, 64, 64, 1, 2, 64, 1, None, None, None, None) == U
    assert lib.wq_int4_fake_quant(None, 9, 4, 64, 64, 1, 1, 32, 1, None, None, None, None) == M_
    assert lib.wq_int4_group_quant_pack(None, 4, 100, 100, 128, None, None, None) == S
    assert lib.wq_int4_group_quant_pack(None, 4, 128, 128, 128, None, None, None) == N_
    assert lib.wq_int4_group_quant_pack_grouped(None, None, 1, 1, 96, None) == U
    assert lib.wq_int4_group_quant_pack_items(None, 5, 128, None) == N_
    assert lib.wq_int4_group_quant_pack_items(None, 5, 96, None) == U
    assert lib.wq_int4_group_quant_pack_items(None, 0, 128, None) == 0
    assert lib.wq_int4_dequant(None, None, None, 4, 100, 128, None) == S
    assert lib.wq_int4_dequant(None, None, None, 4, 128, 12, None) == S
    assert lib.wq_int4_dequant(None, None, None, 4, 128, 128, None) == N_
    assert lib.wq_int4_dequant(None, None, None, 0, 128, 128, None) == 0
    assert lib.wq_int4_dequant_items(None, 3, 128, None) == N_
    assert lib.wq_int4_dequant_items(None, 3, 96, None) == S
    assert lib.wq_int4_dequant_items(None, 0, 128, None) == 0
    assert lib.wq_int4_fake_quant_ste(None, None, 4, 100, 128, 0, None) == S
    assert lib.wq_int4_fake_quant_ste(None, None, 4, 96, 96, 0, None) == U
    assert lib.wq_int4_fake_quant_ste(None, None, 4, 128, 128, 5, None) == M_
    assert lib.wq_int4_fake_quant_ste(None, None, 4, 128, 128, 1, None) == N_
    tlib = wq_testlib.load()
    assert tlib.wq_copy_bytes(None, None, 24, None) == S
    assert tlib.wq_selftest_fp8_elem(0, 0x9000, 0, ctypes.c_void_p(8), None) == S


def test_check_raises_runtime_error():
    with pytest.raises(RuntimeError, match="invalid shape"):
        _lib.check(-2, "probe")


def test_cpu_tensors_are_refused():
    import torch

    import slime_amd

    w = torch.zeros(128, 128, dtype=torch.bfloat16)
    # what is a Triton kernel or a CUDA extension in the reference takes GPU tensors only, there and here
    for fn in (lambda: slime_amd.blockwise_cast_to_fp8_triton(w),
               lambda: slime_amd.pack_layer(w, 128), lambda: slime_amd.fake_int4_quant_cuda(w, (1, 128), True),
               lambda: slime_amd.weight_dequant(w.view(torch.uint8)[:, :128].contiguous(), torch.ones(1, 1))):
        with pytest.raises(RuntimeError, match="GPU"):
            fn()
    # the torch-formulated quantisers take host tensors like the reference's - by way of the GPU, so without one they refuse
    if not torch.cuda.is_available():
        for fn in (lambda: slime_amd.block_fp8(w, (128, 128)), lambda: slime_amd.channel_fp8(w), lambda: slime_amd.tensor_fp8(w)):
            with pytest.raises(RuntimeError, match="GPU"):
                fn()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.WqLibraryError, match="no CPU or pure-torch fallback"):
        _lib.load()


def test_shim_module_does_not_shadow_the_function():
    import slime_amd
    import slime_amd.fake_int4_quant_cuda as shim

    # after the import the package attribute is the module; it must still be callable like the function
    assert callable(slime_amd.fake_int4_quant_cuda) and callable(shim.fake_int4_quant_cuda)
    import torch

    with pytest.raises(RuntimeError):
        slime_amd.fake_int4_quant_cuda(torch.zeros(4, 32), (1, 32), True)      # reaches the function: CPU input refused


def test_top_level_extension_name_resolves_unchanged():
    # the reference's call sites do exactly this (tools/convert_hf_to_int4_direct.py:26, quantizer_compressed_tensors.py:236)
    import importlib
    import sys

    sys.modules.pop("fake_int4_quant_cuda", None)
    mod = importlib.import_module("fake_int4_quant_cuda")
    import slime_amd.int4

    assert mod.fake_int4_quant_cuda is slime_amd.int4.fake_int4_quant_cuda
    assert os.path.dirname(os.path.abspath(mod.__file__)) == ROOT


def test_torch_arithmetic_is_per_thread():
    import threading

    import slime_amd
    from slime_amd import arith

    assert slime_amd.get_torch_arithmetic() == "device"
    seen, go, done = {}, threading.Event(), threading.Event()

    def other():
        seen["before"] = slime_amd.get_torch_arithmetic(), arith.fp8_torch_mode()
        go.wait(5)
        seen["during"] = slime_amd.get_torch_arithmetic(), arith.fp8_torch_mode(), arith.div7_rule()
        with slime_amd.torch_arithmetic("cpu"):
            seen["own"] = slime_amd.get_torch_arithmetic()
        done.set()

    t = threading.Thread(target=other)
    t.start()
    with slime_amd.torch_arithmetic("cpu"):
        assert (slime_amd.get_torch_arithmetic(), arith.fp8_torch_mode(), arith.div7_rule()) == ("cpu", 0, 0)
        with slime_amd.torch_arithmetic("device"):                 # re-entrant
            assert arith.fp8_torch_mode() == 2
        assert arith.fp8_torch_mode() == 0
        go.set()
        assert done.wait(5)
    t.join()
    assert seen == {"before": ("device", 2), "during": ("device", 2, 1), "own": "cpu"}
    assert slime_amd.get_torch_arithmetic() == "device"
    try:                                                            # the process default is what other threads inherit
        slime_amd.set_torch_arithmetic("cpu")
        got = []
        t = threading.Thread(target=lambda: got.append(slime_amd.get_torch_arithmetic()))
        t.start()
        t.join()
        assert got == ["cpu"]
    finally:
        slime_amd.set_torch_arithmetic("device")
    with pytest.raises(ValueError):
        slime_amd.set_torch_arithmetic("gpu")


def test_ue8m0_requests_are_not_ignored():
    import torch

    import slime_amd
    from slime_amd import processors

    assert not processors.ue8m0_requant_enabled()
    with pytest.raises(NotImplementedError, match="TMA"):
        slime_amd.transform_scale_ue8m0(torch.ones(2, 2), mn=256)
    with pytest.raises(AssertionError):
        slime_amd.quant_weight_ue8m0(torch.zeros(128, 128, dtype=torch.bfloat16), [64, 64])
    assert lib_rc("wq_fp8_block_quant", None, 4, 4, 4, 1, None, 4, None, 128, 128, 3, None) == -1      # mode 3 is known
    assert lib_rc("wq_fp8_block_quant_any", None, 1, 4, 4, 4, 1, None, 4, None, 128, 128, 3, None) in (-1, -4)
    assert lib_rc("wq_int4_dequant_any", None, None, 7, None, 4, 8, 8, None) == -3
    assert lib_rc("wq_int4_dequant_any", None, None, 0, None, 4, 8, 3, None) == -2
    assert lib_rc("wq_fp8_bucket_convert", None, 3, None, 128, 128, 1, None) == -1
    assert lib_rc("wq_fp8_bucket_convert_rows_off_lines", None, 3, None, 128, 128, 1, None) == -1
    assert lib_rc("wq_fp8_bucket_convert_rows_off_lines", None, 3, None, 128, 128, 9, None) == -3
    assert lib_rc("wq_int4_bucket_convert", None, 3, None, 48, None) == -4
    assert lib_rc("wq_delta_xor_noalloc", None, None, None, (4 << 30) + 1, 0, None, None) == -6


def lib_rc(name, *args):
    return getattr(_lib.load(), name)(*args)


def test_no_mixed_precision_fma_in_the_dequantiser(tmp_path):
    """`(half)(a * b)` invites the compiler to emit v_fma_mixlo_f16 a, b, 0: one rounding of the exact product where the
    reference rounds to fp32 first, and +0 for a product of -0.  The kernel source blocks that fusion; this compiles the
    file to assembly with the library's own flags and checks that none of it came back."""
    import re
    import shutil
    import subprocess

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    csrc = os.path.join(ROOT, "slime_amd", "csrc")
    flags = re.search(r"^HIPFLAGS \?= (.*?)\n(?!\s)", open(os.path.join(csrc, "Makefile")).read(), re.S | re.M).group(1)
    flags = flags.replace("\\\n", " ").replace("$(ARCH)", "gfx950").split()
    out = tmp_path / "deq.s"
    subprocess.check_call([hipcc, *flags, "-I", os.path.join(ROOT, "include"), "-S", "--cuda-device-only", "-o", str(out),
                           os.path.join(csrc, "wq_fp8_dequant.hip")], stderr=subprocess.DEVNULL)
    asm = out.read_text()
    assert "v_cvt_f16_f32" in asm and "fma_mix" not in asm and "mad_mix" not in asm


def test_no_flat_memory_instruction_in_any_kernel(tmp_path):
    """Every device access goes through a global-address-space pointer.  A pointer that a kernel reads from a descriptor
    table is a generic one to the compiler; one access through it (flat_load / flat_store) is enough for the compiler to
    stop counting outstanding loads in that kernel and wait for all of them (s_waitcnt vmcnt(0)) wherever it waits for
    one - rolling load windows drain after every load and stores go out one round trip at a time.  This compiles every
    kernel source to assembly with the library's own flags and checks that no flat memory instruction is in it."""
    import concurrent.futures
    import glob
    import re
    import shutil
    import subprocess

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    csrc = os.path.join(ROOT, "slime_amd", "csrc")
    flags = re.search(r"^HIPFLAGS \?= (.*?)\n(?!\s)", open(os.path.join(csrc, "Makefile")).read(), re.S | re.M).group(1)
    flags = flags.replace("\\\n", " ").replace("$(ARCH)", "gfx950").split()

    def flat_instructions(src):
        out = tmp_path / (os.path.basename(src) + ".s")
        subprocess.check_call([hipcc, *flags, "-S", "--cuda-device-only", "-o", str(out), src], stderr=subprocess.DEVNULL)
        return src, re.findall(r"^\s*(flat_\w+)", out.read_text(), re.M)

    sources = sorted(glob.glob(os.path.join(csrc, "*.hip")))
    assert len(sources) >= 9
    with concurrent.futures.ThreadPoolExecutor(max_workers=4) as pool:
        for src, found in pool.map(flat_instructions, sources):
            assert not found, f"{os.path.basename(src)}: {len(found)} flat memory instructions ({sorted(set(found))})"


def test_product_never_touches_the_oracle_or_falls_back_to_the_host():
    """The package must not import, load or run anything under oracle/ (test infrastructure), and its entry points must
    refuse to work without the HIP library rather than compute on the host."""
    import glob

    pkg = os.path.join(ROOT, "slime_amd")
    for path in glob.glob(os.path.join(pkg, "**", "*.py"), recursive=True) + [os.path.join(ROOT, "fake_int4_quant_cuda.py")]:
        text = open(path).read()
        assert not re.search(r"^\s*(from|import)\s+oracle\b|libwq_oracle|oracle[/.]", text, re.M), path
    import torch

    import slime_amd

    if not torch.cuda.is_available():
        w = torch.zeros(128, 128, dtype=torch.bfloat16)
        for call in (lambda: slime_amd.block_fp8(w, (128, 128)), lambda: slime_amd.pack_layer(w, 128, True),
                     lambda: slime_amd.weight_dequant(w.view(torch.uint8)[:, :128].view(torch.float8_e4m3fn), torch.ones(1, 1)),
                     lambda: slime_amd.fp8_aligned_weight(w), lambda: slime_amd.delta.checksum("xxh3-128", w)):
            with pytest.raises(RuntimeError):
                call()
