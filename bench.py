"""Benchmark of the weight-conversion hot path on one MI355X.

Headline workload (the "step"): one full weight-sync quantisation pass over a Qwen3-4B-shaped bf16 state
dict - 36 layers x {q [4096,2560], k, v [1024,2560], o [2560,4096], gate, up [9728,2560], down [2560,9728]},
252 tensors, 7.27 GB of bf16 - block-FP8 (128x128, e4m3fn, fp32 scale_inv) with the arithmetic of the
reference's block_fp8, as ONE grouped kernel launch writing into a flat output bucket.  Inputs are resident
in HBM before the timed region; weights are synthetic N(0, 0.02) generated on the device.

Prints ONE JSON line.  `roofline` prices the kernel against the 8 TB/s HBM peak from the algorithmic bytes
(2 B read + 1 B written per element + 4 B of scale per 128x128 block) and the kernel duration measured with
HIP events on the launch stream.  `cpu_baseline` times the CPU restatement of the reference's torch path on
this box's host cores on a bounded sample (one layer's seven tensors, repeated).  `other_workloads` adds the
INT4 pack (Qwen3-30B-A3B experts) and FP8 dequant (DeepSeek-V3 MoE layer) kernels, measured the same way.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

QWEN3_4B_LAYER = [("q_proj", 4096, 2560), ("k_proj", 1024, 2560), ("v_proj", 1024, 2560), ("o_proj", 2560, 4096),
                  ("gate_proj", 9728, 2560), ("up_proj", 9728, 2560), ("down_proj", 2560, 9728)]
QWEN3_4B_LAYERS = 36


def _time_launches(run, steps: int, warmup: int):
    """-> (wall ms per step over the whole timed region, mean per-launch ms from HIP events)."""
    import torch

    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        run()
        ends[i].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev = [s.elapsed_time(e) for s, e in zip(starts, ends)]
    return wall_ms, sum(ev) / len(ev), min(ev)


def _gen_bf16(shape, device, std=0.02, outliers=False):
    import torch

    w = torch.empty(shape, dtype=torch.bfloat16, device=device)
    w.normal_(0.0, std)
    if outliers:
        mask = torch.rand(shape, device=device) < 1e-3
        w[mask] *= 20
    return w


def _traffic_from_profile(name: str):
    """HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, if a summary with a
    `traffic_bytes_per_launch:` line has been committed under profiles/ for this kernel and workload."""
    path = os.path.join(ROOT, "profiles", name)
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    return float(line.split(":", 1)[1].split()[0])
    except OSError:
        pass
    return None


def bench_fp8_quant(dev, steps, warmup):
    import torch

    import slime_amd
    from oracle import c_oracle

    weights, names = [], []
    for layer in range(QWEN3_4B_LAYERS):
        for n, M, N in QWEN3_4B_LAYER:
            weights.append(_gen_bf16((M, N), dev))
            names.append(f"model.layers.{layer}.{n}.weight")
    plan = slime_amd.Fp8QuantPlan(weights, (128, 128))
    wall_ms, ev_ms, ev_min = _time_launches(plan.run, steps, warmup)

    elements = sum(w.numel() for w in weights)
    blocks = plan.total_tiles
    algo_bytes = 3 * elements + 4 * blocks
    bf16_bytes = 2 * elements

    # parity on a sample of the very tensors that were timed
    checked = 0
    for idx in (0, 1, 3, 6, len(weights) - 1):
        q, s = plan.outputs[idx]
        qo, so = c_oracle.fp8_block_quant(weights[idx].cpu(), (128, 128), plan.mode)
        assert torch.equal(q.cpu().view(torch.uint8), qo), f"parity failure on {names[idx]}"
        assert torch.equal(s.cpu().view(torch.int32), so.view(torch.int32)), f"scale parity failure on {names[idx]}"
        checked += 1
    sample = [w.cpu() for w in weights[:len(QWEN3_4B_LAYER)]]
    del plan, weights
    torch.cuda.empty_cache()
    return {
        "wall_ms": wall_ms, "kernel_ms": ev_ms, "kernel_ms_min": ev_min, "elements": elements, "blocks": blocks,
        "algo_bytes": algo_bytes, "bf16_bytes": bf16_bytes, "parity_tensors_checked": checked, "cpu_sample": sample,
    }


def bench_fp8_quant_moe(dev, steps, warmup, layers):
    """Block-FP8 quant of every linear weight of a Qwen3-30B-A3B-shaped state dict (48 layers: 128 experts x
    gate/up [768,2048], down [2048,768]; attention q [4096,2048], k/v [512,2048], o [2048,4096]), one grouped launch."""
    import torch

    import slime_amd
    from oracle import c_oracle

    experts = 128
    weights = []
    for _ in range(layers):
        gate = _gen_bf16((experts, 768, 2048), dev, outliers=True)
        up = _gen_bf16((experts, 768, 2048), dev, outliers=True)
        down = _gen_bf16((experts, 2048, 768), dev, outliers=True)
        for e in range(experts):
            weights += [gate[e], up[e], down[e]]
        weights += [_gen_bf16(sh, dev) for sh in ((4096, 2048), (512, 2048), (512, 2048), (2048, 4096))]
    plan = slime_amd.Fp8QuantPlan(weights, (128, 128))
    wall_ms, ev_ms, ev_min = _time_launches(plan.run, steps, warmup)
    elements = sum(w.numel() for w in weights)
    algo_bytes = 3 * elements + 4 * plan.total_tiles
    for idx in (0, 2, 385, len(weights) - 1):
        q, s = plan.outputs[idx]
        qo, so = c_oracle.fp8_block_quant(weights[idx].cpu().contiguous(), (128, 128), plan.mode)
        assert torch.equal(q.cpu().view(torch.uint8), qo) and torch.equal(s.cpu().view(torch.int32), so.view(torch.int32))
    out = {"workload": f"Qwen3-30B-A3B-shaped state dict, {layers} layers x (128 experts x gate, up [768,2048], down "
                       "[2048,768] + q, k, v, o), block-FP8 128x128, one grouped launch",
           "tensors": len(weights), "bf16_GB": 2 * elements / 1e9, "kernel_ms": ev_ms, "wall_ms": wall_ms,
           "bf16_GBps": 2 * elements / ev_ms / 1e6, "algo_GBps": algo_bytes / ev_ms / 1e6,
           "hbm_frac": algo_bytes / ev_ms / 1e6 / HBM_PEAK_GBS, "parity_tensors_checked": 4}
    del plan, weights
    torch.cuda.empty_cache()
    return out


def bench_int4_pack(dev, steps, warmup, layers):
    import torch

    import slime_amd
    from oracle import c_oracle

    experts = 128
    weights = []
    for _ in range(layers):
        # one allocation per layer and projection; experts are views, as in a grouped-GEMM weight
        gate = _gen_bf16((experts, 768, 2048), dev, outliers=True)
        up = _gen_bf16((experts, 768, 2048), dev, outliers=True)
        down = _gen_bf16((experts, 2048, 768), dev, outliers=True)
        for e in range(experts):
            weights += [gate[e], up[e], down[e]]
    plan = slime_amd.Int4PackPlan(weights, 128)
    wall_ms, ev_ms, ev_min = _time_launches(plan.run, steps, warmup)
    elements = sum(w.numel() for w in weights)
    algo_bytes = elements * 2 + elements // 2 + elements // 128 * 2
    for idx in (0, 2, len(weights) - 1):
        p, s = plan.outputs[idx]
        po, so, _ = c_oracle.int4_pack_layer(weights[idx].cpu().contiguous(), 128, True)
        assert torch.equal(p.cpu(), po) and torch.equal(s.cpu().view(torch.int16), so.view(torch.int16))
    out = {"workload": f"Qwen3-30B-A3B experts, {layers} layers x 128 x (gate, up [768,2048], down [2048,768]), "
                       "INT4 sym group 128, one grouped launch",
           "tensors": len(weights), "bf16_GB": 2 * elements / 1e9, "kernel_ms": ev_ms, "wall_ms": wall_ms,
           "bf16_GBps": 2 * elements / ev_ms / 1e6, "algo_GBps": algo_bytes / ev_ms / 1e6,
           "hbm_frac": algo_bytes / ev_ms / 1e6 / HBM_PEAK_GBS, "parity_tensors_checked": 3}
    del plan, weights
    torch.cuda.empty_cache()
    return out


def bench_int4_inverse(dev, steps, warmup, layers, which):
    """INT4 -> bf16 (`which == "int4deq"`) or the QAT quantise-dequantise forward (`"ste"`) over the expert weights
    of `layers` Qwen3-30B-A3B layers; the 128 experts of a projection are one [128*rows, cols] tensor, one launch
    each (no grouped form exists for these two)."""
    import torch

    import slime_amd
    from oracle import c_oracle

    tensors = []
    for _ in range(layers):
        for rows, cols in ((128 * 768, 2048), (128 * 768, 2048), (128 * 2048, 768)):
            w = _gen_bf16((rows, cols), dev, outliers=True)
            if which == "int4deq":
                p, sc, _ = slime_amd.pack_layer(w, 128, True)
                tensors.append((p, sc, (rows, cols)))
                del w
            else:
                tensors.append(w)
    outs = [None] * len(tensors)
    if which == "int4deq":
        # every expert its own tensor (views of the layer's packed buffer), all of them in one launch
        per_expert = []
        for p, sc, (rows, cols) in tensors:
            r = rows // 128
            per_expert += [(p[e * r:(e + 1) * r], sc[e * r:(e + 1) * r], (r, cols)) for e in range(128)]
        plan = slime_amd.Int4DequantPlan([t[0] for t in per_expert], [t[1] for t in per_expert],
                                         [t[2] for t in per_expert], 128)

        def run():
            plan.run()
    else:
        def run():
            for i, t in enumerate(tensors):
                outs[i] = None          # free the previous output first: the allocator reuses the block
                outs[i] = slime_amd.fake_int4_quantization_ste(t, 128)

    wall_ms, ev_ms, ev_min = _time_launches(run, steps, warmup)
    elements = sum((t[2][0] * t[2][1]) if which == "int4deq" else t.numel() for t in tensors)
    algo_bytes = elements * 2 + elements // 2 + elements // 128 * 2 if which == "int4deq" else elements * 4
    for idx in (0, len(tensors) - 1):
        if which == "int4deq":
            p, sc, shape = tensors[idx]
            want = c_oracle.int4_dequant(p[:1024].cpu(), sc[:1024].cpu(), (1024, shape[1]), 128)
            r = shape[0] // 128
            got = torch.cat([plan.outputs[idx * 128 + e] for e in range(-(-1024 // r))])[:1024]
        else:
            want = c_oracle.int4_fake_ste(tensors[idx][:1024].cpu(), 128, 1)
            got = outs[idx][:1024]
        assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))
    launches = 1 if which == "int4deq" else len(tensors)
    out = {"workload": f"Qwen3-30B-A3B experts, {layers} layers x (gate, up [128x768,2048], down [128x2048,768]), "
                       + ("INT4 group 128 -> bf16" if which == "int4deq" else "INT4 QAT quantise-dequantise forward")
                       + (f", {len(tensors) * 128} expert tensors in one launch" if which == "int4deq"
                          else f", {len(tensors)} launches per step"),
           "launches": launches, "bf16_GB": 2 * elements / 1e9, "kernel_ms": ev_ms, "wall_ms": wall_ms,
           "bf16_GBps": 2 * elements / ev_ms / 1e6, "algo_GBps": algo_bytes / ev_ms / 1e6,
           "hbm_frac": algo_bytes / ev_ms / 1e6 / HBM_PEAK_GBS, "parity_tensors_checked": 2}
    del tensors, outs
    torch.cuda.empty_cache()
    return out


def bench_delta(dev, steps, warmup):
    """Delta weight sync, xor encoding: every linear weight of the Qwen3-4B-shaped state dict against its HBM
    snapshot - diff, changed-byte count, adler32 and snapshot update in one pass per tensor."""
    import numpy as np
    import torch

    from oracle import delta_ref
    from slime_amd import delta

    shapes = [(4096, 2560), (1024, 2560), (1024, 2560), (2560, 4096), (9728, 2560), (9728, 2560), (2560, 9728)] * 36
    news = [_gen_bf16(sh, dev).view(torch.uint8).reshape(-1) for sh in shapes]
    olds = []
    for nw in news:
        old = nw.clone()
        old[:: 3] ^= 1                      # a third of the bytes differ
        olds.append(old)
    check_new, check_old = news[3].cpu().numpy(), olds[3].cpu().numpy().copy()
    diffs, results = delta.xor_diff_many(news, olds, update_snapshot=True)      # the pass whose results are checked
    torch.cuda.synchronize()
    want, changed = delta_ref.xor_delta_ref(check_new, check_old)
    assert np.array_equal(diffs[3].cpu().numpy(), want) and np.array_equal(olds[3].cpu().numpy(), check_new)
    assert results[3].tolist() == [changed, int(delta_ref.adler32_ref(check_new), 16)]
    del diffs

    def run():
        delta.xor_diff_many(news, olds, update_snapshot=True)

    wall_ms, ev_ms, ev_min = _time_launches(run, steps, warmup)
    nbytes = sum(nw.numel() for nw in news)
    out = {"workload": "Qwen3-4B-shaped state dict (252 bf16 tensors, 7.27 GB) against its snapshot in HBM: xor diff, "
                       "changed-byte count, adler32, snapshot update; two launches for the whole bucket",
           "tensors": len(news), "weight_GB": nbytes / 1e9, "kernel_ms": ev_ms, "wall_ms": wall_ms,
           "weight_GBps": nbytes / ev_ms / 1e6, "algo_GBps": 4 * nbytes / ev_ms / 1e6,
           "hbm_frac": 4 * nbytes / ev_ms / 1e6 / HBM_PEAK_GBS, "parity_tensors_checked": 1}
    del news, olds
    torch.cuda.empty_cache()
    return out


def bench_single_tensor_forms(dev, steps, warmup):
    """The per-row / per-tensor FP8 forms and the fake-INT4 quantiser on one vocabulary-sized tensor
    [151936, 2560] bf16 (778 MB), through the Python layer (output allocation included in the timing)."""
    import torch

    import slime_amd
    from oracle import c_oracle

    w = _gen_bf16((151936, 2560), dev, outliers=True)
    el = w.numel()
    head = w[:512].cpu()
    out = {}
    cases = (("fp8_channel_quant", lambda: slime_amd.channel_fp8(w), 3 * el + 4 * w.shape[0]),
             ("fp8_tensor_quant", lambda: slime_amd.tensor_fp8(w), 5 * el),
             ("int4_fake_quant_sym", lambda: slime_amd.fake_int4_quant_cuda(w, (1, 128), True), 4 * el + 4 * el // 128),
             ("int4_fake_quant_asym", lambda: slime_amd.fake_int4_quant_cuda(w, (1, 128), False), 4 * el + 4 * el // 128))
    for name, fn, algo in cases:
        wall_ms, ev_ms, ev_min = _time_launches(fn, steps, warmup)
        out[name] = {"kernel_ms": ev_ms, "bf16_GBps": 2 * el / ev_ms / 1e6, "algo_GBps": algo / ev_ms / 1e6,
                     "hbm_frac": algo / ev_ms / 1e6 / HBM_PEAK_GBS}
    q, s = slime_amd.channel_fp8(w)
    qo, so = c_oracle.fp8_channel_quant(head, 2)
    assert torch.equal(q[:512].cpu().view(torch.uint8), qo) and torch.equal(s[:512].cpu().view(torch.int32), so.view(torch.int32))
    for sym in (True, False):
        q, s, z = slime_amd.fake_int4_quant_cuda(w, (1, 128), sym)
        qo, so, zo = c_oracle.int4_fake_quant(head, (1, 128), sym)
        assert torch.equal(q[:512].cpu().view(torch.int16), qo.view(torch.int16))
        assert torch.equal(s[:512].cpu().view(torch.int16), so.view(torch.int16))
        assert torch.equal(z[:512].cpu().view(torch.int16), zo.view(torch.int16))
    out["workload"] = ("one bf16 [151936, 2560] tensor (778 MB); algorithmic bytes per element: channel 3, tensor 5 (two "
                       "reads), fake INT4 4; parity checked on the first 512 rows")
    del w
    torch.cuda.empty_cache()
    return out


def bench_fp8_dequant(dev, steps, warmup, experts):
    import torch

    import slime_amd
    from oracle import c_oracle

    xs, ss = [], []
    for shape in ((2048, 7168), (2048, 7168), (7168, 2048)):
        codes = torch.randint(0, 254, (experts,) + shape, device=dev, dtype=torch.uint8)
        codes += (codes >= 0x7F).to(torch.uint8)          # uniform over the 254 finite e4m3fn codes
        tm, tn = shape[0] // 128, shape[1] // 128
        sc = torch.exp(torch.empty((experts, tm, tn), device=dev).uniform_(-9.21034, -2.302585))   # log-U[1e-4,1e-1]
        for e in range(experts):
            xs.append(codes[e].view(torch.float8_e4m3fn))
            ss.append(sc[e])
    plan = slime_amd.Fp8DequantPlan(xs, ss, 128, 0, torch.bfloat16)
    wall_ms, ev_ms, ev_min = _time_launches(plan.run, steps, warmup)
    elements = sum(x.numel() for x in xs)
    algo_bytes = 3 * elements + 4 * sum(s.numel() for s in ss)
    for idx in (0, len(xs) - 1):
        yo = c_oracle.fp8_block_dequant(xs[idx].cpu().view(torch.uint8), ss[idx].cpu(), 128, 0)
        assert torch.equal(plan.outputs[idx].cpu().view(torch.int16), yo.view(torch.int16))
    out = {"workload": f"DeepSeek-V3 MoE layer, {experts} experts x (gate, up [2048,7168], down [7168,2048]) e4m3 + "
                       "fp32 scale_inv -> bf16, one grouped launch",
           "tensors": len(xs), "bf16_GB": 2 * elements / 1e9, "kernel_ms": ev_ms, "wall_ms": wall_ms,
           "bf16_GBps": 2 * elements / ev_ms / 1e6, "algo_GBps": algo_bytes / ev_ms / 1e6,
           "hbm_frac": algo_bytes / ev_ms / 1e6 / HBM_PEAK_GBS, "parity_tensors_checked": 2}
    del plan, xs, ss
    torch.cuda.empty_cache()
    return out


def bench_copy(dev, steps, warmup, nbytes=4 << 30):
    """Plain 16-byte-per-lane copy of 4 GiB: known HBM traffic (nbytes read + nbytes written) for scaling the
    FETCH_SIZE / WRITE_SIZE counters, and the practical bandwidth ceiling of this box."""
    import torch

    from slime_amd import _lib

    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 256)
    dst = torch.empty_like(src)

    def run():
        _lib.check(_lib.load().wq_copy_bytes(src.data_ptr(), dst.data_ptr(), nbytes, _lib.stream_ptr(dev)), "copy")

    wall_ms, ev_ms, ev_min = _time_launches(run, steps, warmup)
    assert torch.equal(src[:1 << 20], dst[:1 << 20]) and torch.equal(src[-(1 << 20):], dst[-(1 << 20):])
    return {"workload": "copy_kernel 4 GiB", "bytes_read": nbytes, "bytes_written": nbytes, "kernel_ms": ev_ms,
            "kernel_ms_min": ev_min, "GBps_read_plus_write": 2 * nbytes / ev_ms / 1e6,
            "hbm_frac": 2 * nbytes / ev_ms / 1e6 / HBM_PEAK_GBS}


def bench_stream(dev, n_buckets=64, bucket_bytes=1 << 30, download=True):
    """Host-resident weights: n_buckets x bucket_bytes of bf16 through pinned double buffers -> block-FP8 quant ->
    (optionally) back to pinned host memory.  PCIe-bound by construction; reported next to the kernel-only rate."""
    import torch

    from oracle import c_oracle
    from slime_amd.stream import BucketPipeline, fp8_block_quant_kernel

    N = 4096
    M = bucket_bytes // 2 // N
    pipe = BucketPipeline(dev, fp8_block_quant_kernel(), bucket_bytes, bucket_bytes // 2, 2, depth=2, download=download)
    pipe.time_kernels = True
    for slot in range(2):
        pipe.staging_buffer(slot).copy_(_gen_bf16((M, N), dev).view(-1).view(torch.uint8))
    torch.cuda.synchronize()

    def buckets():
        for i in range(n_buckets):
            yield pipe.staging_buffer(i % 2).view(torch.bfloat16).view(M, N)

    checked = 0
    t0 = time.perf_counter()
    for i, (q, s) in enumerate(pipe.process(buckets())):
        if i == 0 and download:
            qo, so = c_oracle.fp8_block_quant(pipe.staging_buffer(0).view(torch.bfloat16).view(M, N)[:1024], (128, 128), 2)
            assert torch.equal(q[:1024].view(torch.uint8), qo) and torch.equal(s[:8].view(torch.int32), so.view(torch.int32))
            checked = 1
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    total = n_buckets * bucket_bytes
    return {"workload": f"{n_buckets} x {bucket_bytes >> 20} MiB bf16 buckets from pinned host memory -> block-FP8 -> "
                        f"{'pinned host memory' if download else 'device'}, double-buffered",
            "bf16_GB": total / 1e9, "wall_s": wall, "end_to_end_GBps": total / wall / 1e9,
            "kernel_only_GBps": total / (pipe.kernel_ms() / 1e3) / 1e9, "parity_buckets_checked": checked}


def cpu_baseline(sample, budget_s: float):
    """The CPU restatement of the reference torch path (block_fp8 op sequence) on one layer's tensors."""
    import torch

    from oracle import torch_ref

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    nbytes = sum(2 * w.numel() for w in sample)
    for w in sample[1:3]:
        torch_ref.block_fp8_ref(w, (128, 128))      # warm the allocator and thread pool
    reps, t0 = 0, time.perf_counter()
    while True:
        for w in sample:
            torch_ref.block_fp8_ref(w, (128, 128))
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or reps >= 500:
            break
    return {"value": nbytes * reps / dt / 1e9, "unit": "GB/s of bf16 weights", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"layer 0 of the same state dict (7 tensors, {nbytes / 1e6:.0f} MB bf16) x {reps} passes, "
                      f"{dt:.1f} s, torch CPU op-for-op restatement of block_fp8"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="time budget of the CPU baseline sample")
    ap.add_argument("--int4-layers", type=int, default=48, help="layers of Qwen3-30B-A3B experts in the INT4 extra")
    ap.add_argument("--dequant-experts", type=int, default=256)
    ap.add_argument("--no-extras", action="store_true", help="headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--only", choices=["fp8moe", "int4", "dequant", "int4deq", "ste", "delta", "forms", "copy", "stream"], default=None,
                    help="run just one of the other legs and print its record: a kernel for profiling, the plain copy "
                         "kernel that hardware counters are calibrated against, or the host-resident streaming run "
                         "(64 x 1 GiB buckets, PCIe-bound)")
    ap.add_argument("--stream-buckets", type=int, default=64)
    ap.add_argument("--stream-bucket-mib", type=int, default=1024)
    ap.add_argument("--stream-no-download", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures ONE GPU: the path has no cross-GPU exchange and this build has no multi-GPU "
              "launcher; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.manual_seed(0)

    if args.only == "fp8moe":
        print(json.dumps(bench_fp8_quant_moe(dev, args.steps, args.warmup, args.int4_layers)))
        return
    if args.only == "int4":
        print(json.dumps(bench_int4_pack(dev, args.steps, args.warmup, args.int4_layers)))
        return
    if args.only == "dequant":
        print(json.dumps(bench_fp8_dequant(dev, args.steps, args.warmup, args.dequant_experts)))
        return
    if args.only in ("int4deq", "ste"):
        print(json.dumps(bench_int4_inverse(dev, args.steps, args.warmup, min(args.int4_layers, 8), args.only)))
        return
    if args.only == "forms":
        print(json.dumps(bench_single_tensor_forms(dev, args.steps, args.warmup)))
        return
    if args.only == "delta":
        print(json.dumps(bench_delta(dev, args.steps, args.warmup)))
        return
    if args.only == "copy":
        print(json.dumps(bench_copy(dev, args.steps, args.warmup)))
        return
    if args.only == "stream":
        print(json.dumps(bench_stream(dev, args.stream_buckets, args.stream_bucket_mib << 20,
                                      not args.stream_no_download)))
        return

    r = bench_fp8_quant(dev, args.steps, args.warmup)
    achieved = r["algo_bytes"] / r["kernel_ms"] / 1e6      # GB/s
    line = {
        "metric": "GB/s of bf16 weights quantized (FP8 & INT4) + % of HBM peak, 1x MI355X",
        "value": r["bf16_bytes"] / r["wall_ms"] / 1e6,
        "unit": "GB/s of bf16 weights",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": r["wall_ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "Qwen3-4B-shaped bf16 state dict, block-FP8 128x128 quant of all 252 linear weights "
                               "(36 layers x q,k,v,o,gate,up,down; 7.27 GB bf16) = one weight-sync pass, one grouped "
                               "launch, block_fp8 arithmetic as torch evaluates it on GPU tensors",
                   "elements": r["elements"], "blocks": r["blocks"], "bf16_GB": r["bf16_bytes"] / 1e9,
                   "parity_tensors_checked": r["parity_tensors_checked"]},
        "pct_hbm_peak": 100.0 * achieved / HBM_PEAK_GBS,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     "traffic": _traffic_from_profile("fp8_block_quant_qwen3_4b_pmc.txt"),
                     "kernel": "fp8_block_quant_kernel<TORCH_DEVICE, per-tile descriptors>", "kernel_ms": r["kernel_ms"],
                     "kernel_ms_min": r["kernel_ms_min"], "algorithmic_bytes_per_launch": r["algo_bytes"]},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(r["cpu_sample"], args.cpu_seconds)
    else:
        line["cpu_baseline"] = None
    if not args.no_extras:
        extras = {}
        if args.int4_layers > 0:
            extras["fp8_block_quant_moe"] = bench_fp8_quant_moe(dev, args.steps, args.warmup, args.int4_layers)
            extras["int4_group_quant_pack"] = bench_int4_pack(dev, args.steps, args.warmup, args.int4_layers)
        if args.dequant_experts > 0:
            extras["fp8_block_dequant"] = bench_fp8_dequant(dev, args.steps, args.warmup, args.dequant_experts)
        if args.int4_layers > 0:
            extras["int4_dequant"] = bench_int4_inverse(dev, args.steps, args.warmup, min(args.int4_layers, 8), "int4deq")
            extras["int4_qat_forward"] = bench_int4_inverse(dev, args.steps, args.warmup, min(args.int4_layers, 8), "ste")
        extras["delta_xor"] = bench_delta(dev, args.steps, args.warmup)
        extras["single_tensor_forms"] = bench_single_tensor_forms(dev, args.steps, args.warmup)
        line["other_workloads"] = extras
    print(json.dumps(line))


if __name__ == "__main__":
    main()
