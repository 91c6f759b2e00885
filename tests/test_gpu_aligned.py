"""One-pass FP8-aligned weights (quantise to block-FP8 and expand again, in registers) against the two kernels run one
after the other and against the CPU oracle's quantiser followed by its dequantiser."""

import pytest
import torch

import slime_amd
from oracle import c_oracle as C
from slime_amd import _lib
from tests import wq_inputs as I

pytestmark = pytest.mark.gpu
BS = [128, 128]


def _two_pass(w, ue8m0):
    q, s = (slime_amd.quant_weight_ue8m0(w.contiguous(), BS) if ue8m0
            else slime_amd.blockwise_cast_to_fp8_triton(w.contiguous(), (128, 128)))
    return slime_amd.block_quant_dequant(q, s, BS, torch.bfloat16), s


def _oracle(w, mode):
    q, s = C.fp8_block_quant(w, (128, 128), mode)
    return C.fp8_block_dequant(q, s, 128, 0), s


def _same_or_both_nan(a, b):
    an, bn = a.isnan(), b.isnan()
    return bool(torch.equal(an, bn)) and I.same_bits(torch.where(an, torch.zeros_like(a), a),
                                                     torch.where(bn, torch.zeros_like(b), b))


@pytest.mark.parametrize("ue8m0", [False, True])
@pytest.mark.parametrize("shape", [(128, 128), (4096, 4096), (300, 200), (4100, 3000), (7, 7168), (17, 1041), (129, 127),
                                   (1000, 2560)])
def test_aligned_weight_matches_two_pass_and_oracle(cuda, shape, ue8m0):
    w = I.zero_blocks(I.weights(*shape, seed=shape[0] + shape[1]), 0.2, seed=3)
    if shape[0] >= 256 and shape[1] >= 256:
        w[128:256, :128] = I.subnormal_block(seed=5)
        w[:128, 128:256] = I.near_max_block(seed=6)
    y, s = slime_amd.fp8_aligned_weight(w.to(cuda), (128, 128), use_ue8m0=ue8m0, return_scale=True)
    assert y.dtype == torch.bfloat16 and y.shape == w.shape and y.is_contiguous()
    y2, s2 = _two_pass(w.to(cuda), ue8m0)
    assert I.same_bits(y, y2) and I.same_bits(s, s2)
    yo, so = _oracle(w, 3 if ue8m0 else 1)
    assert I.same_bits(y.cpu(), yo) and I.same_bits(s.cpu(), so)
    assert I.same_bits(slime_amd.fp8_aligned_weight(w.to(cuda), use_ue8m0=ue8m0), y)      # without the scale output


def test_aligned_weight_views_and_strides(cuda):
    base = I.weights(512, 776, seed=4).to(cuda)
    for view in (lambda t: t[:, 128:640], lambda t: t.t(), lambda t: t[::2, ::3], lambda t: t[:, 1:769], lambda t: t[3:, :]):
        w = view(base)
        for ue8m0 in (False, True):
            y = slime_amd.fp8_aligned_weight(w, use_ue8m0=ue8m0)
            assert I.same_bits(y, _two_pass(w, ue8m0)[0])
            assert I.same_bits(y.cpu(), _oracle(w.cpu().contiguous(), 3 if ue8m0 else 1)[0])


def test_aligned_weight_every_bf16_value_nan_and_inf(cuda):
    """All 65 536 bit patterns in two blocks (one of them holds the NaNs and infinities: the literal path), then finite
    values only under a spread of block maxima (the fast path)."""
    w = I.all_bf16_values().clone()
    for ue8m0 in (False, True):
        y = slime_amd.fp8_aligned_weight(w.to(cuda), use_ue8m0=ue8m0)
        assert I.same_bits(y, _two_pass(w.to(cuda), ue8m0)[0])            # bit for bit, NaN payloads included
        assert _same_or_both_nan(y.cpu(), _oracle(w, 3 if ue8m0 else 1)[0])
    vals = I.finite_bf16_values()
    g = I.gen(9)
    for ab in torch.randint(1, 0x7F80, (12,), generator=g).tolist() + [0x3F60, 0x7F7F, 1, 0x0080]:
        amax = torch.tensor([ab], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        x = vals[vals.abs() <= amax]
        x = torch.cat([x, torch.zeros((-x.numel()) % (128 * 128), dtype=torch.bfloat16)]).view(-1, 128)
        x[::128, 0] = amax
        for ue8m0 in (False, True):
            y = slime_amd.fp8_aligned_weight(x.to(cuda), use_ue8m0=ue8m0)
            assert I.same_bits(y.cpu(), _oracle(x, 3 if ue8m0 else 1)[0]), (ab, ue8m0)


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
@pytest.mark.parametrize("block", [(128, 128), (64, 32), (128, 256)])
def test_c_abi_all_modes_and_block_shapes(cuda, mode, block):
    """Through the C ABI: every scale rule of the quantiser and block shapes off the tuned path, against the library's
    own two calls (square blocks: the dequantiser's contract) or the oracle."""
    lib = _lib.load()
    w = I.zero_blocks(I.weights(300, 520, seed=mode), 0.2, seed=2, bm=block[0], bn=block[1]).to(cuda)
    M, N = w.shape
    tm, tn = -(-M // block[0]), -(-N // block[1])
    y = torch.empty(M, N, dtype=torch.bfloat16, device=cuda)
    s = torch.empty(tm, tn, dtype=torch.float32, device=cuda)
    st = _lib.stream_ptr(cuda)
    assert lib.wq_fp8_block_quant_dequant(w.data_ptr(), M, N, N, 1, y.data_ptr(), N, s.data_ptr(), block[0], block[1],
                                          mode, st) == 0
    q = torch.empty(M, N, dtype=torch.uint8, device=cuda)
    s2 = torch.empty_like(s)
    assert lib.wq_fp8_block_quant(w.data_ptr(), M, N, N, 1, q.data_ptr(), N, s2.data_ptr(), block[0], block[1], mode, st) == 0
    assert I.same_bits(s, s2)
    # expand the codes with their block's scale on the host: f32(code) * scale, one rounding to bf16
    full = s2.cpu().repeat_interleave(block[0], 0).repeat_interleave(block[1], 1)[:M, :N]
    want = C.f32_to_bf16(C.e4m3fn_to_f32(q.cpu()) * full)
    assert I.same_bits(y.cpu(), want)
    if block[0] == block[1] and mode != 3:
        qo, so = C.fp8_block_quant(w.cpu(), block, mode)
        assert I.same_bits(y.cpu(), C.fp8_block_dequant(qo, so, block[0], 0))


def test_c_abi_argument_checks(cuda):
    lib = _lib.load()
    w = I.weights(128, 128).to(cuda)
    y = torch.empty_like(w)
    st = _lib.stream_ptr(cuda)
    call = lambda *a: lib.wq_fp8_block_quant_dequant(*a, st)
    assert call(w.data_ptr(), 128, 128, 128, 1, y.data_ptr(), 128, None, 128, 128, 9) == -3
    assert call(w.data_ptr(), -1, 128, 128, 1, y.data_ptr(), 128, None, 128, 128, 1) == -2
    assert call(w.data_ptr(), 128, 128, 128, 1, y.data_ptr(), 128, None, 0, 128, 1) == -2
    assert call(None, 128, 128, 128, 1, y.data_ptr(), 128, None, 128, 128, 1) == -1
    assert call(None, 0, 128, 128, 1, None, 128, None, 128, 128, 1) == 0                 # empty: nothing to do
    with pytest.raises(TypeError):
        slime_amd.fp8_aligned_weight(w.float())
    with pytest.raises(ValueError):
        slime_amd.fp8_aligned_weight(w.view(2, 64, 128))
    assert slime_amd.fp8_aligned_weight(w[:0]).shape == (0, 128)


def test_block_quant_dequant_is_weight_dequant_with_explicit_dtype(cuda):
    x = I.fp8_codes(300, 520, seed=1).to(cuda).view(torch.float8_e4m3fn)
    s = I.log_uniform_scales(3, 5, seed=2).to(cuda)
    y = slime_amd.block_quant_dequant(x, s, BS, torch.bfloat16)
    assert I.same_bits(y.cpu(), C.fp8_block_dequant(x.cpu().view(torch.uint8), s.cpu(), 128, 0))
    y32 = slime_amd.block_quant_dequant(x, s, BS, torch.float32)
    full = s.cpu().repeat_interleave(128, 0).repeat_interleave(128, 1)[:300, :520]
    assert I.same_bits(y32.cpu(), C.e4m3fn_to_f32(x.cpu().view(torch.uint8)) * full)
    with pytest.raises(ValueError):
        slime_amd.block_quant_dequant(x, s, [128, 64], torch.bfloat16)


def test_absorb_weight_straight_through_and_cache(cuda):
    lin = torch.nn.Linear(384, 256, bias=False, device=cuda, dtype=torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(I.weights(256, 384, seed=8).to(cuda))
    a = slime_amd.get_fp8_aligned_absorb_weight(lin, use_ue8m0=False)
    assert I.same_bits(a.detach(), _two_pass(lin.weight.detach(), False)[0])
    assert a.requires_grad
    g = I.weights(256, 384, seed=9, std=1.0).to(cuda)
    (a * g).sum().backward()
    assert I.same_bits(lin.weight.grad, g)                        # the gradient passes through unchanged
    cached = lin._sglang_fp8_aligned_absorb_weight_cache
    slime_amd.get_fp8_aligned_absorb_weight(lin, use_ue8m0=False)
    assert lin._sglang_fp8_aligned_absorb_weight_cache is cached  # unchanged weight: no recomputation
    b = slime_amd.get_fp8_aligned_absorb_weight(lin, use_ue8m0=True)
    assert lin._sglang_fp8_aligned_absorb_weight_cache is not cached
    assert I.same_bits(b.detach(), _two_pass(lin.weight.detach(), True)[0])
    with torch.no_grad():
        lin.weight.mul_(2.0)                                      # optimizer step: version counter moves
    c = slime_amd.get_fp8_aligned_absorb_weight(lin, use_ue8m0=False)
    assert I.same_bits(c.detach(), _two_pass(lin.weight.detach(), False)[0])
    slime_amd.set_ue8m0_requant(True)
    try:
        d = slime_amd.get_fp8_aligned_absorb_weight(lin)          # None follows the process switch
    finally:
        slime_amd.set_ue8m0_requant(False)
    assert I.same_bits(d.detach(), _two_pass(lin.weight.detach(), True)[0])
