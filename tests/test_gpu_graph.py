"""The one-launch forms recorded into a HIP graph and replayed: the entry points allocate nothing, clear nothing and
never synchronise, so a weight sync can be captured once and replayed after every optimizer step.  Every replay is
checked - with eager work and synchronisation between the replays - against the eager result on the same inputs."""

import pytest
import torch

import slime_amd
from slime_amd import bucket as B
from slime_amd import delta
from tests import wq_inputs as I
from tests.test_gpu_bucket import FP8_CFG, INT4_CFG, _moe_layer

pytestmark = pytest.mark.gpu


def _capture(fn):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        fn()                                   # warm up on the capture stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    return graph


def _step(tensors, k):
    """An 'optimizer step' done eagerly between replays: the inputs change in place."""
    for i, t in enumerate(tensors):
        t.mul_(1.0 + 0.25 * ((i + k) % 3)).add_(0.001 * k)
    torch.cuda.synchronize()


def test_plans_replay_in_a_graph(cuda):
    ws = [I.weights(m, n, seed=m + n).to(cuda) for m, n in ((256, 384), (128, 256), (300, 520), (768, 2048), (2048, 768))]
    exp = [w for w in ws if w.shape[1] % 128 == 0]
    fp8, int4 = slime_amd.Fp8QuantPlan(ws, (128, 128), mode=1), slime_amd.Int4PackPlan(exp, 128)
    ste = slime_amd.Int4StePlan(exp, 128)

    def run():
        fp8.run(), int4.run(), ste.run()

    graph = _capture(run)
    for k in range(4):
        _step(ws, k)
        for o in (fp8.flat_q, fp8.flat_s, int4.flat_packed, int4.flat_scale, ste.flat_y):
            o.fill_(7)                                             # a replay must rewrite every output
        graph.replay()
        torch.cuda.synchronize()
        for w, (q, s) in zip(ws, fp8.outputs):
            qe, se = slime_amd.blockwise_cast_to_fp8_triton(w, (128, 128))
            assert I.same_bits(q.view(torch.uint8), qe.view(torch.uint8)) and I.same_bits(s, se), k
        for w, (p, s) in zip(exp, int4.outputs):
            pe, se, _ = slime_amd.pack_layer(w, 128, True)
            assert I.same_bits(p, pe) and I.same_bits(s, se), k
        for w, y in zip(exp, ste.outputs):
            assert I.same_bits(y, slime_amd.fake_int4_quantization_ste(w, 128)), k


@pytest.mark.parametrize("cfg", [FP8_CFG, INT4_CFG], ids=["fp8", "int4"])
def test_bucket_convert_replays_in_a_graph(cuda, cfg):
    params = _moe_layer(0, cuda, 100, hidden=256, ffn=384) + _moe_layer(1, cuda, 200, hidden=256, ffn=384)
    conv = B.BucketConverter(None, cfg)
    first = conv.convert(params, bucket_id=0)                      # builds and caches the tables (host work, not captured)
    out = torch.empty_like(first.get_flattened_tensor())
    graph = _capture(lambda: conv.convert(params, out=out, bucket_id=0))
    bf16 = [t for _, cv in params for _, t in cv if t.dtype == torch.bfloat16]
    for k in range(3):
        _step(bf16, k)
        out.fill_(0xAA)
        graph.replay()
        torch.cuda.synchronize()
        want = B.per_param_loop(None, params, cfg)
        got = B.FlattenedBucket(out, first.get_metadata()).reconstruct_tensors()
        assert [n for n, _ in got] == [n for n, _ in want]
        for (n, a), (_, b) in zip(got, want):
            assert I.same_bits(a, b), (n, k)


@pytest.mark.parametrize("with_digest", [False, True])
def test_delta_pass_replays_in_a_graph(cuda, with_digest):
    news = [I.weights(256, 384, seed=1).to(cuda), I.weights(1000, 130, seed=2).to(cuda), I.weights(64, 128, seed=3).to(cuda)]
    olds = [t.clone().view(torch.uint8).flatten() for t in news]          # the snapshot in HBM
    _step(news, 7)
    plan = delta.XorDiffPlan(news, olds, want_diff=True, xxh3=with_digest)
    graph = _capture(lambda: plan.run(update_snapshot=True))
    for k in range(3):
        before = [o.clone() for o in olds]
        _step(news[:2], k)                                                  # the third tensor stays as it is
        graph.replay()
        torch.cuda.synchronize()
        if with_digest:                                                     # the digest of what changed, nothing for the rest
            moved = [not torch.equal(nw.view(torch.uint8).flatten(), ob) for nw, ob in zip(news, before)]
            assert moved[1] and not moved[2], k
            assert plan.hexdigests() == [h if m else None for h, m in zip(delta.xxh3_128_many(news), moved)], k
        for nw, old_before, old_now, diff, res in zip(news, before, olds, plan.diffs, plan.results.cpu()):
            nb = nw.view(torch.uint8).flatten()
            want = nb ^ old_before
            assert torch.equal(diff, want) and torch.equal(old_now, nb), k
            assert int(res[0]) == int((want != 0).sum()), k
