"""The Triton-formulated reference functions as the Triton compiler evaluates them on this GPU, against the HIP
kernels: pins WQ_FP8_MODE_TRITON and weight_dequant to the reference's behaviour on an MI355X."""

import pytest
import torch

import slime_amd
from tests import wq_inputs as I

pytestmark = pytest.mark.gpu
E4M3 = torch.float8_e4m3fn


def _triton_ref():
    try:
        from oracle import triton_ref
    except ImportError as exc:           # no Triton in the image
        pytest.skip(f"triton is not importable: {exc}")
    return triton_ref


def _every_value_blocks(n_amax, seed):
    g = I.gen(seed)
    vals = I.finite_bf16_values()
    rows = []
    for ab in torch.randint(0x0080, 0x7F80, (n_amax,), generator=g).tolist() + [0x2B8D, 0x2EDB, 0x7F7F, 0x0001, 0x0080]:
        amax = torch.tensor([ab], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        x = vals[vals.abs() <= amax][: 128 * 128 * 3]
        x = torch.cat([x, torch.zeros((-x.numel()) % (128 * 128), dtype=torch.bfloat16)]).view(-1, 128)
        x[::128, 0] = amax
        rows.append(x)
    return torch.cat(rows, dim=0)


def _same(q, s, qr, sr):
    assert torch.equal(s.cpu().view(torch.int32), sr.cpu().view(torch.int32))
    a, b = q.cpu().view(torch.uint8), qr.cpu().view(torch.uint8)
    nbad = int((a != b).sum())
    assert nbad == 0, f"{nbad} of {a.numel()} codes differ"


@pytest.mark.parametrize("shape", [(256, 384), (300, 200), (7, 7168), (1024, 2560), (129, 127)])
def test_blockwise_cast_matches_triton_on_this_gpu(cuda, shape):
    T = _triton_ref()
    w = I.zero_blocks(I.weights(*shape, seed=sum(shape)), 0.2, seed=1).to(cuda)
    _same(*slime_amd.blockwise_cast_to_fp8_triton(w, (128, 128)), *T.blockwise_cast_triton_ref(w, (128, 128)))


def test_blockwise_cast_matches_triton_every_bf16_value(cuda):
    T = _triton_ref()
    w = _every_value_blocks(24, seed=5).to(cuda)
    _same(*slime_amd.blockwise_cast_to_fp8_triton(w, (128, 128)), *T.blockwise_cast_triton_ref(w, (128, 128)))


def test_blockwise_cast_scale_for_every_amax(cuda):
    # one block per finite bf16 amax: all 32 640 scales
    T = _triton_ref()
    bits = torch.arange(0, 0x7F80, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    w = torch.zeros(bits.numel(), 32, dtype=torch.bfloat16)
    w[:, 3] = bits
    w[:, 7] = -bits * 0.33
    w = w.to(cuda)
    _same(*slime_amd.blockwise_cast_to_fp8_triton(w, (1, 32)), *T.blockwise_cast_triton_ref(w, (1, 32), num_warps=1))


@pytest.mark.parametrize("shape", [(256, 256), (300, 200), (2048, 7168)])
def test_weight_dequant_matches_triton_on_this_gpu(cuda, shape):
    T = _triton_ref()
    x = I.fp8_codes(*shape, seed=shape[0]).to(cuda).view(E4M3)
    s = I.log_uniform_scales(-(-shape[0] // 128), -(-shape[1] // 128), seed=shape[1]).to(cuda)
    torch.set_default_dtype(torch.bfloat16)
    try:
        got = slime_amd.weight_dequant(x, s)
    finally:
        torch.set_default_dtype(torch.float32)
    assert I.same_bits(got.cpu(), T.weight_dequant_triton_ref(x, s).cpu())
    got32 = slime_amd.weight_dequant(x, s)
    assert I.same_bits(got32.cpu(), T.weight_dequant_triton_ref(x, s, out_dtype=torch.float32).cpu())


@pytest.mark.parametrize("dt", [torch.float16, torch.float32])
def test_blockwise_cast_other_dtypes_match_triton(cuda, dt):
    T = _triton_ref()
    g = torch.Generator().manual_seed(8)
    w = I.zero_blocks(I.weights(300, 1000, seed=9), 0.2, seed=1)
    x = (w.float() * (1 + 1e-3 * torch.randn(300, 1000, generator=g))).to(dt).to(cuda)
    _same(*slime_amd.blockwise_cast_to_fp8_triton(x, (128, 128)), *T.blockwise_cast_triton_ref(x, (128, 128)))
