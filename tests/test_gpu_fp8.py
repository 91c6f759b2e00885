"""HIP FP8 kernels (through the C ABI) against the CPU oracle: bit-exact codes and scales."""

import os

import pytest
import torch

import slime_amd
from oracle import c_oracle as C
from oracle import torch_ref as T
from tests import wq_inputs as I

pytestmark = pytest.mark.gpu
E4M3 = torch.float8_e4m3fn
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _codes(t):
    return t.cpu().view(torch.uint8)


def _bits32(t):
    return t.cpu().contiguous().view(torch.int32)


ARITH = {0: "cpu", 2: "device"}     # oracle mode -> torch arithmetic setting of the host layer
DEFAULT_MODE = 2                    # the host layer's default: torch's GPU evaluation of `/ 448`


def _check_block(w_cpu, w_gpu, block=(128, 128), mode=0):
    if mode == 1:
        q, s = slime_amd.blockwise_cast_to_fp8_triton(w_gpu, block)
    else:
        with slime_amd.torch_arithmetic(ARITH[mode]):
            q, s = slime_amd.block_fp8(w_gpu, block)
    assert q.dtype == E4M3 and q.is_contiguous() and s.dtype == torch.float32
    qo, so = C.fp8_block_quant(w_cpu, block, mode)
    assert q.shape == qo.shape and s.shape == so.shape
    nbad = int((_codes(q) != qo).sum())
    assert nbad == 0, f"{nbad} code mismatches"
    assert torch.equal(_bits32(s), _bits32(so))
    return q, s


SHAPES = [(128, 128), (256, 384), (300, 200), (7, 7168), (1, 1), (1, 8), (129, 127), (4100, 3000), (4096, 4096),
          (1024, 2560), (2560, 9728)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("mode", [0, 1, 2])
def test_block_quant_shapes(cuda, shape, mode):
    w = I.zero_blocks(I.weights(*shape, seed=sum(shape)), 0.2, seed=1)
    _check_block(w, w.to(cuda), mode=mode)


@pytest.mark.parametrize("mode", [0, 2])
def test_block_quant_config1_roundtrip(cuda, mode):
    # [4096,4096] N(0,0.02), 0.1% of entries x20, seed 0: quant then dequant of its own output
    w = I.weights(4096, 4096, seed=0)
    q, s = _check_block(w, w.to(cuda), mode=mode)
    torch.set_default_dtype(torch.bfloat16)
    try:
        d = slime_amd.weight_dequant(q, s)
    finally:
        torch.set_default_dtype(torch.float32)
    assert d.dtype == torch.bfloat16
    assert I.same_bits(d.cpu(), C.fp8_block_dequant(_codes(q), s.cpu(), 128, 0))
    step = s.cpu().repeat_interleave(128, 0).repeat_interleave(128, 1) * 32
    # half an e4m3 step of the block, plus the bf16 rounding of the dequantised value
    assert ((d.cpu().float() - w.float()).abs() <= step / 2 * 1.01 + w.float().abs() * 2.0 ** -7).all()


@pytest.fixture(scope="module")
def tall_ragged():
    # [151937, 2560]: vocabulary-sized, 1-row remainder block row
    return I.zero_blocks(I.weights(151937, 2560, seed=5), 0.2, seed=6)


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_block_quant_tall_ragged(cuda, tall_ragged, mode):
    _check_block(tall_ragged, tall_ragged.to(cuda), mode=mode)


@pytest.mark.parametrize("block", [(32, 32), (64, 128), (128, 64), (1, 128), (16, 48), (256, 256)])
def test_block_quant_other_block_sizes(cuda, block):
    w = I.weights(200, 330, seed=2)
    for mode in (0, 1, 2):
        _check_block(w, w.to(cuda), block, mode)


def test_block_quant_strided_and_unaligned(cuda):
    base = I.weights(512, 776, seed=4)
    bg = base.to(cuda)
    views = [lambda t: t[:, 128:640], lambda t: t.t(), lambda t: t[::2, ::3], lambda t: t[100:357, 5:700],
             lambda t: t[:, 8:], lambda t: t[:, 1:769], lambda t: t[3:, :768]]
    for v in views:
        for mode in (0, 1, 2):
            _check_block(v(base), v(bg), mode=mode)


def test_block_quant_special_blocks(cuda):
    blocks = [I.subnormal_block(seed=1), I.near_max_block(seed=2), I.near_max_block(seed=3, amax=3.0e38),
              I.near_max_block(seed=4, amax=1.2e-38), torch.zeros(128, 128, dtype=torch.bfloat16),
              -torch.zeros(128, 128, dtype=torch.bfloat16)]
    w = torch.cat(blocks, dim=1)
    for mode in (0, 1, 2):
        q, s = _check_block(w, w.to(cuda), mode=mode)
    assert _bits32(s)[0, 4].item() != 0
    # zero block: f32(bf16(1e-12)) / 448, and the same times RN(1/448)
    for arith, bits in (("cpu", 0x27212492), ("device", _zero_block_scale_bits_device())):
        with slime_amd.torch_arithmetic(arith):
            q, s = slime_amd.block_fp8(w.to(cuda), (128, 128))
        assert _bits32(s)[0, 4].item() == bits and (_codes(q)[:, 640:] == 0x80).all()


def _zero_block_scale_bits_device():
    from fractions import Fraction

    from tests import exact_arith as X

    floor_v = Fraction(0x8D | 0x80, 128) * Fraction(2) ** (0x57 - 127)      # bf16 bits 0x2B8D
    v = X.rn_f32(floor_v * X.rn_f32(Fraction(1, 448)))
    return torch.tensor(float(v), dtype=torch.float32).view(torch.int32).item()


def test_block_quant_every_bf16_value(cuda):
    g = I.gen(9)
    amax_bits = torch.cat([torch.randint(1, 0x7F80, (40,), generator=g),
                           torch.tensor([1, 0x2B8C, 0x2B8D, 0x2B8E, 0x7F7F, 0x0080, 0x007F])]).tolist()
    vals = I.finite_bf16_values()
    for ab in amax_bits:
        amax = torch.tensor([ab], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        x = vals[vals.abs() <= amax]
        x = torch.cat([x, torch.zeros((-x.numel()) % (128 * 128), dtype=torch.bfloat16)]).view(-1, 128)
        x[::128, 0] = amax
        for mode in (0, 1, 2):
            _check_block(x, x.to(cuda), mode=mode)


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_block_quant_nan_inf(cuda, mode):
    w = I.weights(128, 384, seed=6)
    w[5, 5] = float("nan")
    w[9, 130] = float("inf")
    w[10, 131] = -float("inf")
    if mode == 1:
        q, s = slime_amd.blockwise_cast_to_fp8_triton(w.to(cuda), (128, 128))
    else:
        with slime_amd.torch_arithmetic(ARITH[mode]):
            q, s = slime_amd.block_fp8(w.to(cuda), (128, 128))
    q, s = _codes(q), s.cpu()
    qo, so = C.fp8_block_quant(w, (128, 128), mode)
    assert s[0, 0].isnan() and ((q[:, :128] & 0x7F) == 0x7F).all()
    assert s[0, 1].isinf()
    nan_o = (qo & 0x7F) == 0x7F
    assert torch.equal((q & 0x7F) == 0x7F, nan_o)
    assert torch.equal(q[~nan_o], qo[~nan_o])
    assert torch.equal(_bits32(s[:, 2]), _bits32(so[:, 2]))


def test_reference_suite_invariants_on_gpu(cuda):
    # the three cases of the reference's tests/test_block_fp8_zero_block.py:38-75
    w = torch.zeros(256, 256, dtype=torch.bfloat16)
    w[0, 0] = 1.0
    q, s = slime_amd.block_fp8(w.to(cuda), (128, 128))
    assert not torch.isnan(q.float()).any() and not torch.isinf(q.float()).any() and (s > 0).all()
    q, s = slime_amd.block_fp8(torch.zeros(128, 128, dtype=torch.bfloat16, device=cuda), (128, 128))
    assert ((q.float() * s.float()) == 0).all()
    torch.manual_seed(0)
    w = torch.randn(256, 256, dtype=torch.float32).to(torch.bfloat16)
    q, s = slime_amd.block_fp8(w.to(cuda), (128, 128))
    deq = q.float().cpu() * s.cpu().repeat_interleave(128, 0).repeat_interleave(128, 1)
    assert not torch.isnan(q.float()).any() and (deq - w.float()).abs().max() < 0.5


def test_reference_suite_on_host_tensors(cuda):
    """The reference's own test file (tests/test_block_fp8_zero_block.py:38-75) hands CPU tensors to block_fp8.  Host tensors
    go through the same kernels in the arithmetic torch uses on CPU tensors and come back on the host: the three cases of
    that file verbatim, the bytes of the CPU oracle (mode 0), and the per-row / per-tensor forms."""
    weight = torch.zeros(256, 256, dtype=torch.bfloat16)
    weight[0, 0] = 1.0
    qweight, scale = slime_amd.block_fp8(weight, (128, 128))
    assert not qweight.is_cuda and not scale.is_cuda and qweight.dtype == torch.float8_e4m3fn
    assert not torch.isnan(qweight.float()).any() and not torch.isinf(qweight.float()).any() and (scale > 0).all()
    assert _bits32(scale)[0, 1].item() == 0x27212492                      # the zero-block scale of the CPU evaluation
    qweight, scale = slime_amd.block_fp8(torch.zeros(128, 128, dtype=torch.bfloat16), (128, 128))
    assert ((qweight.float() * scale.float()) == 0).all()
    torch.manual_seed(0)
    weight = torch.randn(256, 256, dtype=torch.float32).to(torch.bfloat16)
    qweight, scale = slime_amd.block_fp8(weight, (128, 128))
    dequantized = qweight.float() * scale.repeat_interleave(128, dim=0).repeat_interleave(128, dim=1).float()
    assert not torch.isnan(qweight.float()).any() and (dequantized - weight.float()).abs().max() < 0.5
    qo, so = C.fp8_block_quant(weight, (128, 128), 0)
    assert torch.equal(_codes(qweight), qo) and torch.equal(_bits32(scale), _bits32(so))
    w = I.weights(37, 520, seed=4)
    for fn, ora in ((slime_amd.channel_fp8, C.fp8_channel_quant), (slime_amd.tensor_fp8, C.fp8_tensor_quant)):
        q, s = fn(w)
        qo, so = ora(w, 0)
        assert not q.is_cuda and torch.equal(_codes(q), qo) and torch.equal(_bits32(s), _bits32(so))
    q, s = slime_amd.quant_fp8(w, "block", (128, 128))
    assert not q.is_cuda and tuple(s.shape) == (1, 5)
    assert slime_amd.get_torch_arithmetic() == "device"                     # the caller's setting is untouched
    with pytest.raises(RuntimeError, match="GPU"):
        slime_amd.blockwise_cast_to_fp8_triton(w)                           # a Triton kernel in the reference: GPU tensors only


@pytest.mark.parametrize("shape", [(64, 256), (3, 1000), (257, 129), (1024, 2560), (7, 7168), (130, 9728), (5, 20000),
                                   (33, 8200), (1, 8), (300, 16384), (2, 16392)])
def test_channel_and_tensor_quant(cuda, shape):
    w = I.weights(*shape, seed=8)
    w[shape[0] // 2] = 0
    for gpu_fn, ora, sshape in ((slime_amd.channel_fp8, C.fp8_channel_quant, (shape[0], 1)),
                                (slime_amd.tensor_fp8, C.fp8_tensor_quant, (1,))):
        for mode, arith in ARITH.items():
            with slime_amd.torch_arithmetic(arith):
                q, s = gpu_fn(w.to(cuda))
            qo, so = ora(w, mode)
            assert tuple(s.shape) == sshape
            assert torch.equal(_codes(q), qo) and torch.equal(_bits32(s), _bits32(so))
    q, s = slime_amd.quant_fp8(w.to(cuda), "channel")
    assert tuple(s.shape) == (shape[0], 1)
    q, s = slime_amd.quant_fp8(w.to(cuda), "block", (128, 128))
    assert tuple(s.shape) == (-(-shape[0] // 128), -(-shape[1] // 128))


# ------------------------------------------------------------------ dequant

def test_dequant_all_codes(cuda):
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8).repeat(128, 1)
    s = I.log_uniform_scales(1, 2, seed=3)
    for mode, fn in ((0, lambda x, sc: slime_amd.fp8._dequant(x, sc, 128, 0, torch.bfloat16, "t")),
                     (1, slime_amd.weight_dequant_bf16_scale)):
        got = fn(codes.to(cuda).view(E4M3), s.to(cuda)).cpu()
        want = C.fp8_block_dequant(codes, s, 128, mode)
        ok = ~want.isnan()
        assert torch.equal(got.isnan(), want.isnan())
        assert torch.equal(got[ok].view(torch.int16), want[ok].view(torch.int16))


@pytest.mark.parametrize("shape", [(256, 256), (300, 200), (7, 7168), (129, 1), (2048, 7168), (7168, 2048), (16, 1024),
                                   (17, 1040), (5, 1000), (4100, 3000), (151937, 2560)])
def test_dequant_shapes(cuda, shape):
    x = I.fp8_codes(*shape, seed=shape[0])
    s = I.log_uniform_scales(-(-shape[0] // 128), -(-shape[1] // 128), seed=shape[1])
    xg, sg = x.to(cuda).view(E4M3), s.to(cuda)
    y0 = slime_amd.fp8._dequant(xg, sg, 128, 0, torch.bfloat16, "t")
    assert I.same_bits(y0.cpu(), C.fp8_block_dequant(x, s, 128, 0))
    y1 = slime_amd.weight_dequant_bf16_scale(xg, sg)
    assert I.same_bits(y1.cpu(), C.fp8_block_dequant(x, s, 128, 1))
    # default dtype float32 (torch's default): the un-rounded fp32 product, as the reference would give
    y32 = slime_amd.weight_dequant(xg, sg)
    assert y32.dtype == torch.float32
    assert I.same_bits(y32.cpu(), x.view(E4M3).float() * T._expand_scale(s, shape[0], shape[1], 128))


def test_dequant_into_half_precision(cuda):
    """torch's default dtype float16: the reference stores the fp32 product to an fp16 tensor - one RNE rounding, with
    overflow to infinity and gradual underflow (scales up to 1e3 and down to 1e-9 reach both ends)."""
    for shape in ((256, 256), (300, 200), (17, 1040), (5, 1000)):
        x = I.fp8_codes(*shape, seed=shape[0] + 1)
        s = I.log_uniform_scales(-(-shape[0] // 128), -(-shape[1] // 128), seed=shape[1], lo=1e-9, hi=1e3)
        s[0, 0], s[-1, -1] = 1e3, 3e-7                       # overflow to infinity / fp16 subnormals for certain
        torch.set_default_dtype(torch.float16)
        try:
            y = slime_amd.weight_dequant(x.to(cuda).view(E4M3), s.to(cuda))
        finally:
            torch.set_default_dtype(torch.float32)
        want = C.f32_to_f16(C.e4m3fn_to_f32(x) * T._expand_scale(s, shape[0], shape[1], 128))
        assert y.dtype == torch.float16 and I.same_bits(y.cpu(), want)
        assert want.isinf().any() and (want.float().abs() < 6e-5).any()
        # torch's own conversion on the GPU as a second witness
        assert I.same_bits(y, (x.to(cuda).view(E4M3).float() * T._expand_scale(s, shape[0], shape[1], 128).to(cuda)).half())
    with pytest.raises(TypeError):
        slime_amd.fp8._dequant(x.to(cuda).view(E4M3), s.to(cuda), 128, 1, torch.float16, "t")


def test_dequant_reference_kat(cuda):
    # tests/test_hf_to_megatron.py:345-358 of the reference
    w = torch.linspace(-2, 2, 128 * 128).view(128, 128).to(E4M3)
    s = torch.tensor([[2.0]])
    got = slime_amd.weight_dequant_bf16_scale(w.to(cuda), s.to(cuda))
    assert got.dtype == torch.bfloat16 and torch.equal(got.cpu(), w.to(torch.bfloat16) * 2)


def test_dequant_asserts_like_reference(cuda):
    x = I.fp8_codes(128, 256).to(cuda).view(E4M3)
    s = torch.ones(1, 2, device=cuda)
    with pytest.raises(AssertionError):
        slime_amd.weight_dequant(x.t(), s)
    with pytest.raises(AssertionError):
        slime_amd.weight_dequant(x.view(-1), s)


# ------------------------------------------------------------------ grouped launches

def test_quant_plan_equals_single_calls(cuda):
    shapes = [(4096, 2560), (1024, 2560), (1024, 2560), (2560, 4096), (300, 200), (7, 7168), (129, 127), (128, 128)]
    ws = [I.zero_blocks(I.weights(*sh, seed=i), 0.1, seed=i) for i, sh in enumerate(shapes)]
    wg = [w.to(cuda) for w in ws]
    wg[2] = wg[2].t().contiguous().t()      # a strided member: generic path inside the grouped launch
    ws[2] = ws[2]
    assert slime_amd.Fp8QuantPlan(wg[:1], (128, 128)).mode == DEFAULT_MODE
    for mode in (0, 1, 2):
        plan = slime_amd.Fp8QuantPlan(wg, (128, 128), mode)
        outs = plan.run()
        for w, (q, s) in zip(ws, outs):
            qo, so = C.fp8_block_quant(w, (128, 128), mode)
            assert torch.equal(_codes(q), qo) and torch.equal(_bits32(s), _bits32(so))
        # second run after the inputs changed in place: the plan reads current contents
        wg[0].mul_(2)
        outs = plan.run()
        qo, so = C.fp8_block_quant((ws[0].float() * 2).to(torch.bfloat16), (128, 128), mode)
        assert torch.equal(_codes(outs[0][0]), qo) and torch.equal(_bits32(outs[0][1]), _bits32(so))
        wg[0].div_(2)


def test_quant_plan_many_tensors_uses_tile_table(cuda):
    # 8 tensors keep the searched launch (above); 72 mixed tensors get one pre-resolved descriptor per tile
    shapes = [(256, 384), (300, 200), (7, 7168), (129, 127), (128, 128), (1, 1), (640, 128), (100, 1000), (384, 2560)] * 8
    ws = [I.zero_blocks(I.weights(*sh, seed=300 + i), 0.1, seed=i) for i, sh in enumerate(shapes)]
    wg = [w.to(cuda) for w in ws]
    wg[1] = wg[1].t().contiguous().t()              # strided members: generic path behind a tile descriptor
    wg[12] = wg[12].t().contiguous().t()
    for mode in (0, 1, 2):
        plan = slime_amd.Fp8QuantPlan(wg, (128, 128), mode)
        assert plan._tiles is not None and plan._tiles.shape == (plan.total_tiles, 8)
        for w, (q, s) in zip(ws, plan.run()):
            qo, so = C.fp8_block_quant(w, (128, 128), mode)
            assert torch.equal(_codes(q), qo) and torch.equal(_bits32(s), _bits32(so))
    plan = slime_amd.Fp8QuantPlan(wg, (64, 32), 2)   # other block sizes through the same table
    for w, (q, s) in zip(ws, plan.run()):
        qo, so = C.fp8_block_quant(w, (64, 32), 2)
        assert torch.equal(_codes(q), qo) and torch.equal(_bits32(s), _bits32(so))


def test_dequant_plan_equals_single_calls(cuda):
    shapes = [(2048, 7168), (7168, 2048), (300, 200), (16, 1024), (5, 1000)]
    xs = [I.fp8_codes(*sh, seed=i) for i, sh in enumerate(shapes)]
    ss = [I.log_uniform_scales(-(-sh[0] // 128), -(-sh[1] // 128), seed=i) for i, sh in enumerate(shapes)]
    plan = slime_amd.Fp8DequantPlan([x.to(cuda).view(E4M3) for x in xs], [s.to(cuda) for s in ss])
    for x, s, y in zip(xs, ss, plan.run()):
        assert I.same_bits(y.cpu(), C.fp8_block_dequant(x, s, 128, 0))


# ------------------------------------------------------------------ full-size configurations

def test_qwen3_4b_layer_all_linears(cuda):
    # one decoder layer of the Qwen3-4B-shaped state dict (q, k, v, o, gate, up, down), grouped launch
    shapes = {"q": (4096, 2560), "k": (1024, 2560), "v": (1024, 2560), "o": (2560, 4096),
              "gate": (9728, 2560), "up": (9728, 2560), "down": (2560, 9728)}
    ws = {n: I.weights(*sh, seed=100 + i, outlier_p=0) for i, (n, sh) in enumerate(shapes.items())}
    outs = slime_amd.block_fp8_many([w.to(cuda) for w in ws.values()], (128, 128))
    for (n, w), (q, s) in zip(ws.items(), outs):
        qo, so = C.fp8_block_quant(w, (128, 128), DEFAULT_MODE)
        assert torch.equal(_codes(q), qo) and torch.equal(_bits32(s), _bits32(so)), n


def test_golden_fixtures(cuda):
    from safetensors.torch import load_file

    f = load_file(os.path.join(GOLDEN, "fp8_golden.safetensors"))
    for case in sorted({k.split("/")[0] for k in f}):
        w = f[f"{case}/w"]
        for arith, tag in (("cpu", "block"), ("device", "block_dev")):
            with slime_amd.torch_arithmetic(arith):
                q, s = slime_amd.block_fp8(w.to(cuda), (128, 128))
            assert torch.equal(_codes(q), f[f"{case}/q_{tag}"].view(torch.uint8)), (case, arith)
            assert torch.equal(_bits32(s), _bits32(f[f"{case}/s_{tag}"])), (case, arith)
        q, s = slime_amd.blockwise_cast_to_fp8_triton(w.to(cuda), (128, 128))
        assert torch.equal(_codes(q), f[f"{case}/q_cast"].view(torch.uint8)), case
        assert torch.equal(_bits32(s), _bits32(f[f"{case}/s_cast"])), case
        d = slime_amd.fp8._dequant(f[f"{case}/q_block"].to(cuda), f[f"{case}/s_block"].to(cuda), 128, 0,
                                   torch.bfloat16, "golden")
        assert I.same_bits(d.cpu(), f[f"{case}/deq"]), case


# ------------------------------------------------------------------ torch's own GPU kernels as a second witness

def test_torch_evaluates_scalar_division_as_reciprocal_multiply_on_gpu(cuda):
    # the premise of the "device" arithmetic: for every finite positive bf16 amax, torch's GPU `t / 448` and
    # `t / 7` are t * RN(1/448) and t * RN(1/7), and differ from the CPU results somewhere
    t = torch.arange(0, 0x7F80, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    for d in (448.0, 7):
        on_gpu = (t.to(cuda) / d).cpu()
        inv = (torch.ones((), dtype=torch.float32) / d).item()
        assert I.same_bits(on_gpu, t * inv)
        assert not I.same_bits(on_gpu, t / d)


def _every_value_blocks(n_amax, seed):
    g = I.gen(seed)
    vals = I.finite_bf16_values()
    rows = []
    for ab in torch.randint(0x0080, 0x7F80, (n_amax,), generator=g).tolist() + [0x2B8D, 0x7F7F, 0x0001]:
        amax = torch.tensor([ab], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        x = vals[vals.abs() <= amax][: 128 * 128 * 3]
        x = torch.cat([x, torch.zeros((-x.numel()) % (128 * 128), dtype=torch.bfloat16)]).view(-1, 128)
        x[::128, 0] = amax
        rows.append(x)
    return torch.cat(rows, dim=0)


def test_torch_ops_on_the_gpu_agree_with_the_kernels(cuda):
    # the reference's own op sequence, executed by torch on the GPU, against the HIP kernels in "device" arithmetic
    ws = [I.zero_blocks(I.weights(300, 200, seed=21), 0.2, seed=2), I.weights(1024, 2560, seed=22),
          _every_value_blocks(12, seed=23)]
    for w in ws:
        wg = w.to(cuda)
        for ref, mine in ((lambda x: T.block_fp8_ref(x, (128, 128)), lambda x: slime_amd.block_fp8(x, (128, 128))),
                          (T.channel_fp8_ref, slime_amd.channel_fp8), (T.tensor_fp8_ref, slime_amd.tensor_fp8)):
            qr, sr = ref(wg)
            q, s = mine(wg)
            assert torch.equal(_bits32(s), _bits32(sr))
            assert torch.equal(_codes(q), _codes(qr))


def test_channel_and_tensor_quant_views_and_specials(cuda):
    base = I.weights(300, 4104, seed=31)
    base[5, 100] = float("nan")
    base[9, 7] = float("inf")
    base[11] = 0
    base[12] = -0.0
    base[13, :2048] = I.subnormal_block(1, 2048, seed=3)[0]
    bg = base.to(cuda)
    views = [lambda t: t, lambda t: t[:, 8:4104], lambda t: t[:, :4096], lambda t: t[::2], lambda t: t[:, 4:],
             lambda t: t.t(), lambda t: t[20:], lambda t: t[20:, :2048]]
    for v in views:
        for mode, arith in ARITH.items():
            with slime_amd.torch_arithmetic(arith):
                q, s = slime_amd.channel_fp8(v(bg))
            qo, so = C.fp8_channel_quant(v(base), mode)
            so_c, s_c = so, s.cpu()
            assert torch.equal(s_c.isnan(), so_c.isnan())
            ok = ~so_c.isnan().view(-1)
            assert torch.equal(_bits32(s_c)[ok], _bits32(so_c)[ok])
            qc = _codes(q)
            nan_o = (qo & 0x7F) == 0x7F
            assert torch.equal((qc & 0x7F) == 0x7F, nan_o) and torch.equal(qc[~nan_o], qo[~nan_o])
    clean = I.weights(256, 4096, seed=32)
    for v in (lambda t: t, lambda t: t[:, 8:], lambda t: t[::2], lambda t: t.t()):
        for mode, arith in ARITH.items():
            with slime_amd.torch_arithmetic(arith):
                q, s = slime_amd.tensor_fp8(v(clean.to(cuda)))
            qo, so = C.fp8_tensor_quant(v(clean), mode)
            assert torch.equal(_codes(q), qo) and torch.equal(_bits32(s), _bits32(so))
    with_nan = clean.clone()
    with_nan[3, 3] = float("nan")
    q, s = slime_amd.tensor_fp8(with_nan.to(cuda))
    assert s.isnan().all() and ((_codes(q) & 0x7F) == 0x7F).all()


def test_channel_quant_every_bf16_value(cuda):
    rows = []
    vals = I.finite_bf16_values()
    g = I.gen(17)
    for ab in torch.randint(1, 0x7F80, (20,), generator=g).tolist() + [0x2B8C, 0x2B8D, 0x7F7F, 1]:
        amax = torch.tensor([ab], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        x = vals[vals.abs() <= amax][:4096 * 3]
        x = torch.cat([x, torch.zeros((-x.numel()) % 4096, dtype=torch.bfloat16)]).view(-1, 4096)
        x[:, 0] = amax
        rows.append(x)
    w = torch.cat(rows)
    for mode, arith in ARITH.items():
        with slime_amd.torch_arithmetic(arith):
            q, s = slime_amd.channel_fp8(w.to(cuda))
        qo, so = C.fp8_channel_quant(w, mode)
        assert torch.equal(_codes(q), qo) and torch.equal(_bits32(s), _bits32(so))


# ------------------------------------------------------------------ fp16 / fp32 weights

@pytest.mark.parametrize("dt", [torch.float16, torch.float32])
@pytest.mark.parametrize("mode", [0, 1, 2])
def test_block_quant_other_dtypes(cuda, dt, mode):
    g = torch.Generator().manual_seed(4)
    for shape in ((256, 384), (300, 200), (7, 7168), (129, 127), (1024, 2560)):
        w = I.zero_blocks(I.weights(*shape, seed=sum(shape)), 0.2, seed=1)
        x = (w.float() * (1 + 1e-3 * torch.randn(shape, generator=g))).to(dt)
        for view in (lambda t: t, lambda t: t.t(), lambda t: t[::2, 1:]):
            xc, xg = view(x), view(x.to(cuda))
            if mode == 1:
                q, s = slime_amd.blockwise_cast_to_fp8_triton(xg, (128, 128))
            else:
                with slime_amd.torch_arithmetic(ARITH[mode]):
                    q, s = slime_amd.block_fp8(xg, (128, 128))
            qo, so = C.fp8_block_quant(xc, (128, 128), mode)
            qc = _codes(q)
            nan = (qo & 0x7F) == 0x7F
            assert torch.equal((qc & 0x7F) == 0x7F, nan) and torch.equal(qc[~nan], qo[~nan])
            assert torch.equal(_bits32(s), _bits32(so))


@pytest.mark.parametrize("dt", [torch.float16, torch.float32])
def test_block_quant_other_dtypes_match_torch_ops_on_the_gpu(cuda, dt):
    g = torch.Generator().manual_seed(5)
    w = I.weights(512, 640, seed=6)
    x = (w.float() * (1 + 1e-3 * torch.randn(512, 640, generator=g))).to(dt).to(cuda)
    q, s = slime_amd.block_fp8(x, (128, 128))
    qr, sr = T.block_fp8_ref(x, (128, 128))
    assert torch.equal(_bits32(s), _bits32(sr)) and torch.equal(_codes(q), _codes(qr))


@pytest.mark.parametrize("dt", [torch.float16, torch.float32])
@pytest.mark.parametrize("mode", [0, 2])
def test_channel_and_tensor_quant_other_dtypes(cuda, dt, mode):
    """fp16 / fp32 weights through the per-row and per-tensor forms, against the oracle: the per-tensor quotient is
    rounded to the weight's dtype (twice-rounded for fp16, once for fp32), rows are blocks of one row."""
    g = torch.Generator().manual_seed(7)
    for shape in ((256, 384), (300, 200), (7, 7168), (129, 127)):
        w = I.weights(*shape, seed=sum(shape))
        x = (w.float() * (1 + 1e-3 * torch.randn(shape, generator=g))).to(dt)
        x[3] = 0                                            # an all-zero row: 0 / 0 for fp16 (its clamp bound rounds to 0)
        for view in (lambda t: t, lambda t: t.t(), lambda t: t[::2, 1:]):
            xc, xg = view(x), view(x.to(cuda))
            with slime_amd.torch_arithmetic(ARITH[mode]):
                q, s = slime_amd.channel_fp8(xg)
                qt, st = slime_amd.tensor_fp8(xg)
            for (got, sc), (qo, so) in (((q, s), C.fp8_channel_quant(xc, mode)), ((qt, st), C.fp8_tensor_quant(xc, mode))):
                qc = _codes(got)
                nan = (qo & 0x7F) == 0x7F
                assert torch.equal((qc & 0x7F) == 0x7F, nan) and torch.equal(qc[~nan], qo[~nan]), (shape, dt, mode)
                snan = so.isnan()
                assert torch.equal(sc.cpu().isnan().view(-1), snan.view(-1))
                assert torch.equal(_bits32(sc).view(-1)[~snan.view(-1)], _bits32(so).view(-1)[~snan.view(-1)])
            assert s.shape == (xg.shape[0], 1) and st.shape == (1,)


@pytest.mark.parametrize("dt", [torch.float16, torch.float32])
def test_channel_and_tensor_quant_other_dtypes_match_torch_ops_on_the_gpu(cuda, dt):
    # torch's own GPU kernels running the reference's lines: the witness for the dtype of the quotient and of the divisor
    g = torch.Generator().manual_seed(8)
    for shape, std in (((512, 640), 0.02), ((300, 200), 1.0), ((64, 4096), 1e-3)):
        w = I.weights(*shape, seed=9, std=std)
        x = (w.float() * (1 + 1e-3 * torch.randn(shape, generator=g))).to(dt).to(cuda)
        for ref, mine in ((T.channel_fp8_ref, slime_amd.channel_fp8), (T.tensor_fp8_ref, slime_amd.tensor_fp8)):
            qr, sr = ref(x)
            q, s = mine(x)
            assert torch.equal(_bits32(s), _bits32(sr)) and torch.equal(_codes(q), _codes(qr)), (shape, dt)


def test_int8_weights_are_refused(cuda):
    with pytest.raises(TypeError):
        slime_amd.block_fp8(torch.zeros(128, 128, dtype=torch.int8, device=cuda), (128, 128))


def test_grouped_search_entry_point(cuda):
    # Fp8QuantPlan uses the per-tile table; the descriptor-array + prefix-sum form stays part of the C ABI
    from slime_amd import _lib

    shapes = [(4096, 2560), (300, 200), (7, 7168), (129, 127), (1024, 2560)]
    ws = [I.zero_blocks(I.weights(*sh, seed=60 + i), 0.1, seed=i) for i, sh in enumerate(shapes)]
    wg = [w.to(cuda) for w in ws]
    wg[1] = wg[1].t().contiguous().t()
    outs, rows, starts, tiles = [], [], [0], 0
    for w in wg:
        M, N = w.shape
        q = torch.empty(M, N, dtype=torch.uint8, device=cuda)
        sc = torch.empty(-(-M // 128), -(-N // 128), dtype=torch.float32, device=cuda)
        outs.append((q, sc))
        rows.append([w.data_ptr(), q.data_ptr(), sc.data_ptr(), M, N, w.stride(0), w.stride(1), N])
        tiles += sc.numel()
        starts.append(tiles)
    descs = torch.tensor(rows, dtype=torch.int64).to(cuda)
    st = torch.tensor(starts, dtype=torch.int64).to(cuda)
    for mode in (0, 1, 2):
        rc = _lib.load().wq_fp8_block_quant_grouped(descs.data_ptr(), st.data_ptr(), len(ws), tiles, 128, 128, mode,
                                                    _lib.stream_ptr(cuda))
        _lib.check(rc, "grouped")
        for w, (q, sc) in zip(ws, outs):
            qo, so = C.fp8_block_quant(w, (128, 128), mode)
            assert torch.equal(q.cpu(), qo) and torch.equal(_bits32(sc), _bits32(so))
