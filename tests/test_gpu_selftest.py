"""Exhaustive on-device checks of the shortcuts the production kernels take (GPU only).

The kernels replace the reference's per-element IEEE division by a reciprocal + two-FMA refinement and
its software casts by gfx950 conversion instructions.  Each shortcut is compared with the literal
arithmetic over its complete input domain."""

import pytest
import torch

import wq_testlib
from slime_amd import _lib

pytestmark = pytest.mark.gpu


def _run(fn, *args):
    out = torch.zeros(2, dtype=torch.int64, device="cuda")
    rc = fn(*args, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "selftest")
    torch.cuda.synchronize()
    count, first = out.tolist()
    return count, first & 0xFFFFFFFFFFFFFFFF


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_fp8_element_function_whole_domain(cuda, mode):
    # every finite bf16 amax x every bf16 x with |x| <= amax: 2^31 pairs
    count, first = _run(wq_testlib.load().wq_selftest_fp8_elem, 0, 0x7F80, mode)
    assert count == 0, f"{count} mismatches, first at amax=0x{first >> 16:04x} x=0x{first & 0xFFFF:04x}"


def test_int4_element_function_whole_domain(cuda):
    count, first = _run(wq_testlib.load().wq_selftest_int4_elem, 0, 0x7F80)
    assert count == 0, f"{count} mismatches, first at amax=0x{first >> 16:04x} x=0x{first & 0xFFFF:04x}"


def test_hw_fp32_to_e4m3_all_inputs(cuda):
    count, first = _run(wq_testlib.load().wq_selftest_cvt_fp8, 0, 1 << 32)
    assert count == 0, f"{count} mismatches, first at fp32 bits 0x{first:08x}"


def test_hw_fp32_to_bf16_all_inputs(cuda):
    count, first = _run(wq_testlib.load().wq_selftest_cvt_bf16, 0, 1 << 32)
    assert count == 0, f"{count} mismatches, first at fp32 bits 0x{first:08x}"


def test_hw_e4m3_to_fp32_all_codes(cuda):
    count, first = _run(wq_testlib.load().wq_selftest_decode_fp8)
    assert count == 0, f"{count} mismatches, first code 0x{first:02x}"


def test_copy_kernel(cuda):
    g = torch.Generator().manual_seed(0)
    src = torch.randint(0, 256, (1 << 20,), generator=g, dtype=torch.int32).to(torch.uint8).cuda()
    dst = torch.zeros_like(src)
    _lib.check(wq_testlib.load().wq_copy_bytes(src.data_ptr(), dst.data_ptr(), src.numel(),
                                         torch.cuda.current_stream().cuda_stream), "copy")
    assert torch.equal(src, dst)


@pytest.mark.parametrize("ratio, piece", [(2, 16384), (4, 8192)])
def test_fold_stream_kernel(cuda, ratio, piece):
    """The compute-free R:1 stream the benchmark uses as this box's ceiling for the quantisers' read:write mixes: every output
    piece is the xor of R consecutive input pieces."""
    g = torch.Generator().manual_seed(ratio)
    n_out = 16384 * 37
    src = torch.randint(0, 256, (ratio * n_out,), generator=g, dtype=torch.int32).to(torch.uint8).cuda()
    dst = torch.zeros(n_out, dtype=torch.uint8, device="cuda")
    lib = wq_testlib.load()
    _lib.check(lib.wq_stream_fold_bytes(src.data_ptr(), dst.data_ptr(), n_out, ratio, torch.cuda.current_stream().cuda_stream), "fold")
    pieces = src.view(-1, ratio, piece)
    want = pieces[:, 0].clone()
    for r in range(1, ratio):
        want ^= pieces[:, r]
    assert torch.equal(dst, want.reshape(-1))
    assert lib.wq_stream_fold_bytes(src.data_ptr(), dst.data_ptr(), n_out, 3, None) == -3          # mode
    assert lib.wq_stream_fold_bytes(src.data_ptr(), dst.data_ptr(), n_out + 16, ratio, None) == -2  # shape
    assert lib.wq_stream_fold_bytes(src.data_ptr() + 8, dst.data_ptr(), n_out, ratio, None) == -5   # alignment


@pytest.mark.parametrize("writes", [2, 4])
def test_expand_stream_kernel(cuda, writes):
    """The compute-free 1:W stream (the dequantisers' mixes): output piece w of every 4 KiB input piece is the input with w added
    to each dword."""
    g = torch.Generator().manual_seed(writes)
    n_in = 16384 * 37
    src = torch.randint(-2 ** 31, 2 ** 31 - 1, (n_in // 4,), generator=g, dtype=torch.int32).cuda()
    dst = torch.zeros(writes * n_in // 4, dtype=torch.int32, device="cuda")
    lib = wq_testlib.load()
    _lib.check(lib.wq_stream_expand_bytes(src.data_ptr(), dst.data_ptr(), n_in, writes, torch.cuda.current_stream().cuda_stream), "expand")
    want = src.view(-1, 1, 1024) + torch.arange(writes, dtype=torch.int32, device="cuda").view(1, writes, 1)
    assert torch.equal(dst, want.reshape(-1))
    assert lib.wq_stream_expand_bytes(src.data_ptr(), dst.data_ptr(), n_in, 3, None) == -3           # mode
    assert lib.wq_stream_expand_bytes(src.data_ptr(), dst.data_ptr(), n_in + 4096, writes, None) == -2  # shape
    assert lib.wq_stream_expand_bytes(src.data_ptr() + 8, dst.data_ptr(), n_in, writes, None) == -5   # alignment


def test_empty_launch(cuda):
    lib = wq_testlib.load()
    _lib.check(lib.wq_empty_launch(1024, 256, torch.cuda.current_stream().cuda_stream), "empty launch")
    torch.cuda.synchronize()
    assert lib.wq_empty_launch(0, 256, None) == -2 and lib.wq_empty_launch(4, 2048, None) == -2
