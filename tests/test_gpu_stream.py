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
