"""One tensor with more than 2^31 elements (more than 4 GiB of bf16): every index that is 32 bits wide inside a kernel
must be relative to a 64-bit origin.  [70000, 32768]: element 2^31 is the first of row 65536, the last block row has 112
rows.  The oracle runs on row stripes of the very tensor that was processed (block rows, groups and rows are
independent): the first rows, the rows on both sides of element 2^31, and the ragged end."""

import zlib

import pytest
import torch

import slime_amd
from oracle import c_oracle as C
from slime_amd import arith, delta
from tests import wq_inputs as I

pytestmark = pytest.mark.gpu
M, N = 70000, 32768
STRIPES = [(0, 128), (65408, 65664), (69888, 70000)]          # block-row aligned


@pytest.fixture(scope="module")
def big(cuda):
    g = torch.Generator(device=cuda).manual_seed(11)
    w = torch.empty((M, N), dtype=torch.bfloat16, device=cuda).normal_(0.0, 0.02, generator=g)
    w[65536, :8] = torch.tensor([3.0, -3.0, 0.5, -0.0, 1e-30, 2.0, -1.0, 0.25], dtype=torch.bfloat16)   # around element 2^31
    yield w
    del w
    torch.cuda.empty_cache()


def _stripes(w):
    return [(a, b, w[a:b].cpu()) for a, b in STRIPES]


def test_fp8_block_quant_dequant_and_aligned(cuda, big):
    for fn, mode in ((slime_amd.block_fp8, arith.fp8_torch_mode()), (slime_amd.blockwise_cast_to_fp8_triton, 1)):
        q, s = fn(big, (128, 128))
        for a, b, wc in _stripes(big):
            qo, so = C.fp8_block_quant(wc, (128, 128), mode)
            assert torch.equal(q[a:b].cpu().view(torch.uint8), qo), (mode, a)
            assert I.same_bits(s[a // 128:-(-b // 128)].cpu(), so), (mode, a)
    y = slime_amd.block_quant_dequant(q, s, [128, 128], torch.bfloat16)
    y1 = slime_amd.fp8_aligned_weight(big)
    for a, b, wc in _stripes(big):
        want = C.fp8_block_dequant(q[a:b].cpu().view(torch.uint8), s[a // 128:-(-b // 128)].cpu(), 128, 0)
        assert I.same_bits(y[a:b].cpu(), want) and I.same_bits(y1[a:b].cpu(), want), a
    assert torch.equal(y.view(torch.int16), y1.view(torch.int16))          # the whole tensor, on the GPU


def test_fp8_row_and_tensor_forms(cuda, big):
    mode = arith.fp8_torch_mode()
    q, s = slime_amd.channel_fp8(big)
    for a, b, wc in _stripes(big):
        qo, so = C.fp8_channel_quant(wc, mode)
        assert torch.equal(q[a:b].cpu().view(torch.uint8), qo) and I.same_bits(s[a:b].cpu(), so), a
    q, s = slime_amd.tensor_fp8(big)
    top = big.view(-1)[big.abs().view(-1).argmax()].reshape(1, 1).cpu()     # the element that sets the scale
    for a, b, wc in _stripes(big):
        probe = torch.cat([wc, top.expand(1, N)])                            # same amax as the whole tensor
        qo, so = C.fp8_tensor_quant(probe, mode)
        assert torch.equal(q[a:b].cpu().view(torch.uint8), qo[:-1]) and I.same_bits(s.cpu(), so.view(1)), a


def test_int4_forms(cuda, big):
    p, s, _ = slime_amd.pack_layer(big, 128, True)
    d = slime_amd.dequantize_int4(p, s, torch.tensor([M, N]), 128)
    y = slime_amd.fake_int4_quantization_ste(big, 128)
    for a, b, wc in _stripes(big):
        po, so, _ = C.int4_pack_layer(wc, 128, True)
        assert torch.equal(p[a:b].cpu(), po) and I.same_bits(s[a:b].cpu(), so), a
        assert I.same_bits(d[a:b].cpu(), C.int4_dequant(po, so, (b - a, N), 128)), a
        assert I.same_bits(y[a:b].cpu(), C.int4_fake_ste(wc, 128, arith.div7_rule())), a
    del p, s, d, y
    for sym in (True, False):
        q, s, z = slime_amd.fake_int4_quant_cuda(big, (1, 128), sym)
        for a, b, wc in _stripes(big):
            qo, so, zo = C.int4_fake_quant(wc, (1, 128), sym)
            assert I.same_bits(q[a:b].cpu(), qo) and I.same_bits(s[a:b].cpu(), so) and I.same_bits(z[a:b].cpu(), zo), (sym, a)
        del q, s, z
    big8 = big[:69888]                                                       # asymmetric packing needs M % 8 == 0
    p, s, zp = slime_amd.pack_layer(big8, 128, False)
    for a, b in ((0, 128), (65408, 65664), (69760, 69888)):
        po, so, zo = C.int4_pack_layer(big8[a:b].cpu(), 128, False)
        assert torch.equal(p[a:b].cpu(), po) and I.same_bits(s[a:b].cpu(), so), a
        assert torch.equal(zp[:, a // 8:b // 8].cpu(), zo), a


def test_delta_pass_over_more_than_4_gib(cuda, big):
    old = torch.zeros(big.numel() * 2, dtype=torch.uint8, device=cuda)
    old[: 1 << 20] = big.view(torch.uint8).view(-1)[: 1 << 20]             # the first MiB is unchanged
    diff, result = delta.xor_diff(big, old, update_snapshot=True)
    nb = big.view(torch.uint8).view(-1)
    assert torch.equal(old, nb)                                              # snapshot updated
    assert not diff[: 1 << 20].any() and torch.equal(diff[1 << 20:], nb[1 << 20:])
    changed, adler = result.cpu().tolist()
    assert changed == int((nb[1 << 20:] != 0).sum())
    host = nb.cpu().numpy()
    want = 1
    for i in range(0, host.size, 1 << 30):
        want = zlib.adler32(host[i:i + (1 << 30)], want)
    assert adler == want
    assert delta.checksum("adler32", big) == f"{want:08x}"


def test_digest_from_the_delta_pass_over_more_than_4_gib(cuda, big):
    """4.27 GiB in one tensor: 4.5 M XXH3 blocks summed by the diff kernel and walked in one chain, against the stand-alone
    digest kernels and the xxhash package on the host."""
    xxhash = pytest.importorskip("xxhash")
    nb = big.view(torch.uint8).view(-1)
    old = nb.clone()
    old[123456789] ^= 0x40                                                   # one byte differs: the tensor counts as changed
    _, results, digests = delta.xor_diff_many([big], [old], update_snapshot=True, want_diff=False, xxh3=True)
    assert results[0, 0].item() == 1 and torch.equal(old, nb)
    got = delta._hex128(*digests[0].tolist())
    assert got == delta.xxh3_128(big)
    hasher = xxhash.xxh3_128()
    host = nb.cpu().numpy()
    for i in range(0, host.size, 1 << 30):
        hasher.update(host[i:i + (1 << 30)])
    assert got == hasher.hexdigest()
