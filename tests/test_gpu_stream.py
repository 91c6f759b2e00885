"""Host-resident buckets through the double-buffered pipeline: outputs equal the oracle, bucket by bucket."""

import pytest
import torch

from oracle import c_oracle as C
from slime_amd.stream import BucketPipeline, fp8_block_quant_kernel, int4_pack_kernel
from tests import wq_inputs as I

pytestmark = pytest.mark.gpu


def test_stream_fp8_ragged_buckets(cuda):
    shapes = [(512, 1024), (300, 1000), (1024, 512), (7, 7168), (640, 768), (512, 1024), (128, 128)]
    ws = [I.weights(*sh, seed=i) for i, sh in enumerate(shapes)]
    pipe = BucketPipeline(cuda, fp8_block_quant_kernel(), max(w.numel() for w in ws) * 2,
                          max(w.numel() for w in ws), 2, depth=2)
    n = 0
    for w, (q, s) in zip(ws, pipe.process(iter(ws))):
        qo, so = C.fp8_block_quant(w, (128, 128), 2)
        assert q.device.type == "cpu" and torch.equal(q.view(torch.uint8), qo)
        assert torch.equal(s.view(torch.int32), so.view(torch.int32))
        n += 1
    assert n == len(ws)


def test_stream_int4_and_no_download(cuda):
    ws = [I.weights(256, 1024, seed=10 + i) for i in range(5)]
    pipe = BucketPipeline(cuda, int4_pack_kernel(128), 256 * 1024 * 2, 256 * 1024 // 2, 2, depth=3, download=False)
    outs = []
    for packed, scale in pipe.process(iter(ws)):
        assert packed.is_cuda
        outs.append((packed.cpu(), scale.cpu()))
    for w, (p, s) in zip(ws, outs):
        po, so, _ = C.int4_pack_layer(w, 128, True)
        assert torch.equal(p, po) and I.same_bits(s, so)


def test_stream_rejects_oversized_and_gpu_buckets(cuda):
    pipe = BucketPipeline(cuda, fp8_block_quant_kernel(), 1024, 512, 2)
    with pytest.raises(ValueError):
        list(pipe.process([torch.zeros(64, 64, dtype=torch.bfloat16)]))
    with pytest.raises(ValueError):
        list(pipe.process([torch.zeros(16, 16, dtype=torch.bfloat16, device=cuda)]))


def _stripe_rows(M, seed, n=4):
    """First, last and a few seeded 128-row stripes of an [M, N] bucket."""
    g = I.gen(seed)
    picks = {0, (M - 1) // 128} | set(torch.randint(0, -(-M // 128), (n,), generator=g).tolist())
    return [(b * 128, min(M, b * 128 + 128)) for b in sorted(picks)]


def _check_fp8_stripes(w_bucket, q, s, seed):
    M = w_bucket.shape[0]
    for r0, r1 in _stripe_rows(M, seed):
        qo, so = C.fp8_block_quant(w_bucket[r0:r1], (128, 128), 2)
        assert torch.equal(q[r0:r1].view(torch.uint8), qo), (seed, r0)
        assert torch.equal(s[r0 // 128].view(torch.int32), so[0].view(torch.int32)), (seed, r0)


def test_stream_holds_previous_result_and_refills_staging(cuda):
    # every bucket is written into the pipeline's own staging buffer right before it is handed over (different data
    # each time), and every result is checked one advance AFTER it was yielded: the documented buffer lifetimes
    M, N, n_buckets = 1024, 2048, 7
    base = I.weights(M, N, seed=40).view(torch.int16)
    pipe = BucketPipeline(cuda, fp8_block_quant_kernel(), M * N * 2, M * N, 2, depth=2)
    sent = []

    def buckets():
        for i in range(n_buckets):
            stage = pipe.staging_buffer(i % 2)[:M * N * 2].view(torch.int16).view(M, N)
            stage.copy_(base ^ (5 * i))                   # low mantissa bits differ from bucket to bucket
            sent.append(stage.clone().view(torch.bfloat16))
            yield stage.view(torch.bfloat16)

    held = None
    n = 0
    for k, out in enumerate(pipe.process(buckets())):
        if held is not None:
            qo, so = C.fp8_block_quant(sent[k - 1], (128, 128), 2)
            assert torch.equal(held[0].view(torch.uint8), qo), k - 1
            assert torch.equal(held[1].view(torch.int32), so.view(torch.int32)), k - 1
        held = out
        n += 1
    qo, so = C.fp8_block_quant(sent[-1], (128, 128), 2)
    assert n == n_buckets and torch.equal(held[0].view(torch.uint8), qo)


def test_stream_one_gib_buckets(cuda):
    # the bucketed-streaming row of the edge-case configuration at its real bucket size: 1 GiB of bf16 per bucket from
    # pinned host memory, a handful of buckets (every staging and output slot is reused), sampled stripes against
    # the oracle; stops at the first mismatch
    N = 4096
    M = (1 << 30) // 2 // N
    n_buckets = 5
    base = I.weights(M // 16, N, seed=41).view(torch.int16).repeat(16, 1)
    pipe = BucketPipeline(cuda, fp8_block_quant_kernel(), 1 << 30, 1 << 29, 2, depth=2)

    def buckets():
        for i in range(n_buckets):
            stage = pipe.staging_buffer(i % 2).view(torch.int16).view(M, N)
            torch.bitwise_xor(base, 3 * i + 1, out=stage)
            yield stage.view(torch.bfloat16)

    n = 0
    for i, (q, s) in enumerate(pipe.process(buckets())):
        assert q.shape == (M, N) and s.shape == (M // 128, N // 128)
        expect = (base ^ (3 * i + 1)).view(torch.bfloat16)         # rebuilt: the staging buffer has moved on
        _check_fp8_stripes(expect, q, s, seed=i)
        n += 1
    assert n == n_buckets
