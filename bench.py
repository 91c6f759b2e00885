"""Benchmark of the low-precision weight-conversion path on one MI355X.

`python bench.py --gpus 1 --steps K --warmup W` prints ONE JSON line.  A step is one conversion pass over a
Qwen3-30B-A3B-shaped bf16 state dict resident in HBM into BOTH rollout formats: block-FP8 128x128 of all 18 624 linear
weights (one grouped launch), then symmetric group-128 INT4 pack of the 18 432 expert weights (one grouped launch).
`value` = bf16 bytes quantised per second over the timed region (wall clock around K steps); `roofline` describes the
kernel of the step with the LOWER fraction of the HBM peak (both are listed under `roofline_kernels`), from its
algorithmic bytes and its mean launch time measured with HIP events on the launch stream.  `cpu_baseline` times the
CPU restatement of the reference's torch path on this box's host cores on bounded samples of the same tensors (the
mix of the step, and per leg).  `other_workloads` holds the remaining configurations (Qwen3-4B state dict, the
[4096,4096] matrix, FP8 -> bf16 of a DeepSeek-V3 layer, INT4 -> bf16, the QAT forward, delta sync, single-tensor forms
and the bucket-level weight-sync drop-in), measured the same way.
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
if os.path.join(ROOT, "tests") not in sys.path:
    sys.path.append(os.path.join(ROOT, "tests"))         # wq_testlib: the binding of the calibration kernels

HBM_PEAK_GBS = 8000.0
HEADLINE_FP8_MODE = 0          # WQ_FP8_MODE_TORCH: block_fp8 as the reference's test and the CPU baseline evaluate it

QWEN3_4B_LAYER = [("q_proj", 4096, 2560), ("k_proj", 1024, 2560), ("v_proj", 1024, 2560), ("o_proj", 2560, 4096),
                  ("gate_proj", 9728, 2560), ("up_proj", 9728, 2560), ("down_proj", 2560, 9728)]
QWEN3_4B_LAYERS = 36


def _time_step(runs, steps: int, warmup: int):
    """A step = the callables of `runs` in order.  -> (wall ms per step over the whole timed region, [mean ms per run],
    [min ms per run]); the per-run times come from HIP events recorded on the current stream around each run."""
    import torch

    for _ in range(warmup):
        for run in runs:
            run()
    torch.cuda.synchronize()
    marks = [[torch.cuda.Event(enable_timing=True) for _ in range(len(runs) + 1)] for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        marks[i][0].record()
        for k, run in enumerate(runs):
            run()
            marks[i][k + 1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    per = [[m[k].elapsed_time(m[k + 1]) for m in marks] for k in range(len(runs))]
    return wall_ms, [sum(v) / len(v) for v in per], [min(v) for v in per]


def _time_launches(run, steps: int, warmup: int):
    """-> (wall ms per step over the whole timed region, mean per-launch ms from HIP events, min)."""
    wall_ms, mean, mn = _time_step([run], steps, warmup)
    return wall_ms, mean[0], mn[0]


def _time_back_to_back(run, launches: int, rounds: int = 5):
    """`launches` calls of `run` in a row between ONE pair of HIP events, `rounds` times -> median microseconds per
    launch.  This is what a loop of per-tensor calls pays per call; an event pair around every single launch adds the
    cost of the two event packets to each measurement."""
    import torch

    per = []
    for _ in range(rounds):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(launches):
            run()
        b.record()
        torch.cuda.synchronize()
        per.append(a.elapsed_time(b) * 1e3 / launches)
    per.sort()
    return per[len(per) // 2]


def _gen_bf16(shape, device, std=0.02, outliers=False):
    import torch

    w = torch.empty(shape, dtype=torch.bfloat16, device=device)
    w.normal_(0.0, std)
    if outliers:
        mask = torch.rand(shape, device=device) < 1e-3
        w[mask] *= 20
    return w


def kernel_source_hash(*files: str) -> str:
    """sha256 over the named files of slime_amd/csrc (a kernel's source and the shared header)."""
    import hashlib

    h = hashlib.sha256()
    for f in files:
        with open(os.path.join(ROOT, "slime_amd", "csrc", f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


KERNEL_SOURCES = {
    "fp8_block_quant": ("wq_fp8_quant.hip", "wq_common.h"),
    "int4_pack": ("wq_int4.hip", "wq_common.h"),
    "fp8_block_dequant": ("wq_fp8_dequant.hip", "wq_common.h"),
    "int4_dequant": ("wq_int4_dequant.hip", "wq_common.h"),
    "delta_xor": ("wq_delta.hip", "wq_common.h", "wq_xxh3_common.h"),
    "fp8_fake_quant": ("wq_fp8_fake.hip", "wq_common.h"),
}


def _traffic_from_profile(name: str, kernel: str):
    """HBM bytes per launch that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE measured for this kernel and workload, from
    the summary committed under profiles/ - a separate run, not this one.  The summary records the sha256 of the
    kernel's source; when the source has changed since, the figure is stale and is NOT reported.
    -> (bytes or None, note)."""
    path = os.path.join(ROOT, "profiles", name)
    traffic = recorded = None
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    traffic = float(line.split(":", 1)[1].split()[0])
                elif line.startswith("kernel_source_sha256:"):
                    recorded = line.split(":", 1)[1].split()[0]
    except OSError:
        return None, f"profiles/{name} not found"
    if traffic is None:
        return None, f"profiles/{name} holds no traffic figure"
    current = kernel_source_hash(*KERNEL_SOURCES[kernel])
    if recorded != current:
        return None, (f"profiles/{name} was taken on another version of the kernel source "
                      f"(recorded {str(recorded)[:12]}, now {current[:12]}): figure withheld")
    return traffic, f"profiles/{name} (rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE, separate run; kernel source {current[:12]} unchanged since)"


def _moe_state_dict(dev, layers, experts=128):
    """Qwen3-30B-A3B-shaped linear weights: per layer 128 experts x (gate, up [768,2048], down [2048,768]) as views of
    one allocation per projection (the layout of a grouped-GEMM weight), plus q [4096,2048], k, v [512,2048],
    o [2048,4096].  -> (all weights in state-dict order, the expert weights only)."""
    weights, expert_weights = [], []
    for _ in range(layers):
        gate = _gen_bf16((experts, 768, 2048), dev, outliers=True)
        up = _gen_bf16((experts, 768, 2048), dev, outliers=True)
        down = _gen_bf16((experts, 2048, 768), dev, outliers=True)
        for e in range(experts):
            expert_weights += [gate[e], up[e], down[e]]
            weights += [gate[e], up[e], down[e]]
        weights += [_gen_bf16(sh, dev) for sh in ((4096, 2048), (512, 2048), (512, 2048), (2048, 4096))]
    return weights, expert_weights


def bench_north_star(dev, steps, warmup, layers):
    """One conversion pass over the Qwen3-30B-A3B-shaped state dict into both formats: block-FP8 of every linear
    weight, then INT4 pack of the expert weights.  Two grouped launches per step."""
    import torch

    import slime_amd
    from oracle import c_oracle

    weights, expert_weights = _moe_state_dict(dev, layers)
    # The headline computes block_fp8 as the reference's own test runs it and as the CPU baseline beside it does: torch's
    # CPU evaluation (WQ_FP8_MODE_TORCH = 0).  The two other arithmetic variants are timed on the same tensors below.
    fp8_plan = slime_amd.Fp8QuantPlan(weights, (128, 128), mode=HEADLINE_FP8_MODE)
    int4_plan = slime_amd.Int4PackPlan(expert_weights, 128)
    wall_ms, mean, mn = _time_step([fp8_plan.run, int4_plan.run], steps, warmup)

    el_fp8 = sum(w.numel() for w in weights)
    el_int4 = sum(w.numel() for w in expert_weights)
    algo_fp8 = 3 * el_fp8 + 4 * fp8_plan.total_tiles
    algo_int4 = 2 * el_int4 + el_int4 // 2 + el_int4 // 128 * 2
    fp8_sample = (0, 2, 385, len(weights) - 1)

    def check_fp8(plan):
        for idx in fp8_sample:
            q, s = plan.outputs[idx]
            qo, so = c_oracle.fp8_block_quant(weights[idx].cpu().contiguous(), (128, 128), plan.mode)
            assert torch.equal(q.cpu().view(torch.uint8), qo), f"FP8 parity failure on tensor {idx} (mode {plan.mode})"
            assert torch.equal(s.cpu().view(torch.int32), so.view(torch.int32)), f"FP8 scale parity failure on tensor {idx} (mode {plan.mode})"
        return len(fp8_sample)

    # parity on a sample of the very tensors that were timed
    checked = check_fp8(fp8_plan)
    for idx in (0, 2, len(expert_weights) - 1):
        p, s = int4_plan.outputs[idx]
        po, so, _ = c_oracle.int4_pack_layer(expert_weights[idx].cpu().contiguous(), 128, True)
        assert torch.equal(p.cpu(), po), f"INT4 parity failure on tensor {idx}"
        assert torch.equal(s.cpu().view(torch.int16), so.view(torch.int16)), f"INT4 scale parity failure on tensor {idx}"
        checked += 1
    out = {"wall_ms": wall_ms, "layers": layers, "tensors_fp8": len(weights), "tensors_int4": len(expert_weights),
           "bf16_bytes": 2 * (el_fp8 + el_int4), "parity_tensors_checked": checked,
           "fp8": {"kernel_ms": mean[0], "kernel_ms_min": mn[0], "elements": el_fp8, "blocks": fp8_plan.total_tiles,
                   "algo_bytes": algo_fp8, "mode": fp8_plan.mode},
           "int4": {"kernel_ms": mean[1], "kernel_ms_min": mn[1], "elements": el_int4, "algo_bytes": algo_int4}}
    del fp8_plan, int4_plan
    torch.cuda.empty_cache()
    # the FP8 launch of the step in the two other arithmetic variants, same tensors, each checked against the oracle in
    # its own mode: 1 = the weight-sync cast (blockwise_cast_to_fp8_triton), 2 = block_fp8 as torch evaluates it on GPU tensors
    modes = {}
    for mode, label in ((1, "weight-sync cast: fp32 amax floored at 1e-10, x * (1 / scale)"),
                        (2, "block_fp8 as torch evaluates it on GPU tensors: scale = amax * RN(1/448), IEEE x / scale")):
        plan = slime_amd.Fp8QuantPlan(weights, (128, 128), mode=mode)
        _, ev_ms, ev_min = _time_launches(plan.run, steps, warmup)
        n = check_fp8(plan)
        modes[str(mode)] = {"arithmetic": label, "kernel_ms": ev_ms, "kernel_ms_min": ev_min,
                            "hbm_frac": algo_fp8 / ev_ms / 1e6 / HBM_PEAK_GBS, "parity_tensors_checked": n}
        del plan
        torch.cuda.empty_cache()
    modes[str(HEADLINE_FP8_MODE)] = {"arithmetic": "block_fp8 as torch evaluates it on CPU tensors (the headline): scale = amax / 448, IEEE x / scale",
                                     "kernel_ms": mean[0], "kernel_ms_min": mn[0],
                                     "hbm_frac": algo_fp8 / mean[0] / 1e6 / HBM_PEAK_GBS, "parity_tensors_checked": len(fp8_sample)}
    out["fp8_modes"] = modes
    del weights, expert_weights
    torch.cuda.empty_cache()
    return out


def bench_fp8_quant(dev, steps, warmup):
    """Block-FP8 quant of every linear weight of a Qwen3-4B-shaped state dict (252 tensors, 7.27 GB), one launch."""
    import torch

    import slime_amd
    from oracle import c_oracle

    weights = [_gen_bf16((M, N), dev) for _ in range(QWEN3_4B_LAYERS) for _, M, N in QWEN3_4B_LAYER]
    plan = slime_amd.Fp8QuantPlan(weights, (128, 128))
    wall_ms, ev_ms, ev_min = _time_launches(plan.run, steps, warmup)
    elements = sum(w.numel() for w in weights)
    algo_bytes = 3 * elements + 4 * plan.total_tiles
    for idx in (0, 1, 3, 6, len(weights) - 1):      # parity on a sample of the very tensors that were timed
        q, s = plan.outputs[idx]
        qo, so = c_oracle.fp8_block_quant(weights[idx].cpu(), (128, 128), plan.mode)
        assert torch.equal(q.cpu().view(torch.uint8), qo) and torch.equal(s.cpu().view(torch.int32), so.view(torch.int32))
    traffic, note = _traffic_from_profile("fp8_block_quant_qwen3_4b.txt", "fp8_block_quant")
    out = {"workload": "Qwen3-4B-shaped bf16 state dict, block-FP8 128x128 quant of all 252 linear weights (36 layers x "
                       "q,k,v,o,gate,up,down), one grouped launch, block_fp8 arithmetic as torch evaluates it on GPU tensors",
           "tensors": len(weights), "bf16_GB": 2 * elements / 1e9, "kernel_ms": ev_ms, "kernel_ms_min": ev_min,
           "wall_ms": wall_ms, "bf16_GBps": 2 * elements / ev_ms / 1e6, "algo_GBps": algo_bytes / ev_ms / 1e6,
           "hbm_frac": algo_bytes / ev_ms / 1e6 / HBM_PEAK_GBS, "algorithmic_bytes_per_launch": algo_bytes,
           "traffic": traffic, "traffic_source": note, "parity_tensors_checked": 5}
    del plan, weights
    torch.cuda.empty_cache()
    return out


def bench_cfg1(dev, steps, warmup, n_buffers=8):
    """The single [4096, 4096] matrix (N(0, 0.02), 0.1 % of entries x20): block-FP8 quant then dequant of its own
    output.  One 100 MB round trip fits the last-level cache, so the timed loop cycles through `n_buffers` distinct
    matrices (cold) and, separately, re-runs one (warm)."""
    import torch

    import slime_amd
    import wq_testlib
    from oracle import c_oracle
    from slime_amd import _lib

    lib = _lib.load()
    M = N = 4096
    g = torch.Generator().manual_seed(0)
    w0 = torch.randn(M, N, generator=g) * 0.02
    w0[torch.rand(M, N, generator=g) < 0.001] *= 20
    w0 = w0.to(torch.bfloat16)
    ws = [w0.to(dev)] + [_gen_bf16((M, N), dev, outliers=True) for _ in range(n_buffers - 1)]
    qs = [torch.empty((M, N), dtype=torch.uint8, device=dev) for _ in ws]
    ss = [torch.empty((M // 128, N // 128), dtype=torch.float32, device=dev) for _ in ws]
    ys = [torch.empty((M, N), dtype=torch.bfloat16, device=dev) for _ in ws]
    mode = HEADLINE_FP8_MODE
    st = _lib.stream_ptr(dev)
    state = {"i": 0}

    def quant(k):
        _lib.check(lib.wq_fp8_block_quant(ws[k].data_ptr(), M, N, N, 1, qs[k].data_ptr(), N, ss[k].data_ptr(), 128, 128,
                                          mode, st), "cfg1 quant")

    def dequant(k):
        _lib.check(lib.wq_fp8_block_dequant(qs[k].data_ptr(), ss[k].data_ptr(), ys[k].data_ptr(), _lib.DTYPE_BF16, M, N,
                                            128, _lib.DEQ_MODE_F32SCALE, st), "cfg1 dequant")

    def cold_quant():
        state["i"] = (state["i"] + 1) % n_buffers
        quant(state["i"])

    def cold_dequant():
        dequant(state["i"])

    wall_c, mean_c, _ = _time_step([cold_quant, cold_dequant], max(steps, 2 * n_buffers), max(warmup, n_buffers))
    wall_w, mean_w, _ = _time_step([lambda: quant(0), lambda: dequant(0)], max(steps, 2 * n_buffers), warmup)
    # the same launches back to back (the shape of a per-tensor loop), and what an empty launch costs both ways
    state["i"] = 0

    def cold_dequant_next():
        state["i"] = (state["i"] + 1) % n_buffers
        dequant(state["i"])

    q_b2b = _time_back_to_back(cold_quant, 8 * n_buffers)
    d_b2b = _time_back_to_back(cold_dequant_next, 8 * n_buffers)
    tl = wq_testlib.load()

    def empty():
        _lib.check(tl.wq_empty_launch(1024, 256, st), "empty launch")

    _, empty_mean, _ = _time_step([empty], max(steps, 2 * n_buffers), warmup)
    empty_b2b = _time_back_to_back(empty, 8 * n_buffers)
    qo, so = c_oracle.fp8_block_quant(w0, (128, 128), mode)
    assert torch.equal(qs[0].cpu(), qo) and torch.equal(ss[0].cpu().view(torch.int32), so.view(torch.int32))
    yo = c_oracle.fp8_block_dequant(qo, so, 128, 0)
    assert torch.equal(ys[0].cpu().view(torch.int16), yo.view(torch.int16))
    algo = 3 * M * N + 4 * (M // 128) * (N // 128)
    out = {"workload": f"one bf16 [4096,4096] matrix, block-FP8 quant then dequant of its own output; cold = {n_buffers} "
                       "distinct matrices cycled, warm = the same matrix every step; whole tensor checked against the oracle",
           "quant_kernel_ms_cold": mean_c[0], "dequant_kernel_ms_cold": mean_c[1],
           "quant_kernel_ms_warm": mean_w[0], "dequant_kernel_ms_warm": mean_w[1],
           "quant_hbm_frac_cold": algo / mean_c[0] / 1e6 / HBM_PEAK_GBS,
           "dequant_hbm_frac_cold": algo / mean_c[1] / 1e6 / HBM_PEAK_GBS,
           "back_to_back": {"what": "64 launches in a row between one pair of events (a per-tensor loop), cold buffers; "
                                    "microseconds per launch",
                            "quant_us_cold": q_b2b, "dequant_us_cold": d_b2b,
                            "quant_hbm_frac_cold": algo / q_b2b / 1e3 / HBM_PEAK_GBS,
                            "dequant_hbm_frac_cold": algo / d_b2b / 1e3 / HBM_PEAK_GBS},
           "empty_launch_us": {"what": "an empty kernel of 1024 workgroups x 256 lanes: the launch floor under both ways of timing",
                               "event_pair_per_launch": empty_mean[0] * 1e3, "back_to_back": empty_b2b},
           "mode": mode,
           "roundtrip_bf16_GBps_cold": 2 * M * N / (mean_c[0] + mean_c[1]) / 1e6,
           "roundtrip_bf16_GBps_warm": 2 * M * N / (mean_w[0] + mean_w[1]) / 1e6,
           "note": "32 MiB tensors, one wave of workgroups: the *_kernel_ms_* figures bracket every launch with its own event "
                   "pair and so contain the cost of the event packets (compare empty_launch_us); warm runs are served "
                   "from the last-level cache, so their rate is not an HBM figure"}
    del ws, qs, ss, ys
    torch.cuda.empty_cache()
    return out


def bench_launch_sizes(dev, shapes=((2048, 2048), (4096, 4096), (8192, 4096), (8192, 8192), (16384, 8192), (32768, 8192),
                                    (65536, 8192), (131072, 8192))):
    """How the achieved fraction of the HBM peak grows with the size of ONE launch: a single bf16 matrix through
    wq_fp8_block_quant and its codes through wq_fp8_block_dequant, launches back to back over enough distinct buffers
    to stay out of the last-level cache.  Every launch pays a fixed cost - the gap between two kernels on a stream,
    the first bytes' latency, the tail in which the last workgroups drain - that only multi-gigabyte launches
    amortise; the sub-millisecond legs of this benchmark sit on this curve."""
    import torch

    import wq_testlib
    from slime_amd import _lib

    lib, tl = _lib.load(), wq_testlib.load()
    st = _lib.stream_ptr(dev)
    empty_b2b = _time_back_to_back(lambda: tl.wq_empty_launch(1024, 256, st), 64)
    rows = []
    for M, N in shapes:
        touched = 2 * (3 * M * N)                                   # bytes of one quant + one dequant
        n = max(2, min(16, (600 << 20) // touched + 1))             # >= 600 MB cycled, or two buffers of the largest
        ws = [torch.empty((M, N), dtype=torch.bfloat16, device=dev).normal_(0, 0.02) for _ in range(n)]
        qs = [torch.empty((M, N), dtype=torch.uint8, device=dev) for _ in ws]
        ss = [torch.empty((M // 128, N // 128), dtype=torch.float32, device=dev) for _ in ws]
        ys = [torch.empty((M, N), dtype=torch.bfloat16, device=dev) for _ in ws]
        k = {"i": 0}

        def quant():
            k["i"] = (k["i"] + 1) % n
            i = k["i"]
            _lib.check(lib.wq_fp8_block_quant(ws[i].data_ptr(), M, N, N, 1, qs[i].data_ptr(), N, ss[i].data_ptr(), 128, 128,
                                              HEADLINE_FP8_MODE, st), "quant")

        def dequant():
            k["i"] = (k["i"] + 1) % n
            i = k["i"]
            _lib.check(lib.wq_fp8_block_dequant(qs[i].data_ptr(), ss[i].data_ptr(), ys[i].data_ptr(), _lib.DTYPE_BF16, M, N,
                                                128, _lib.DEQ_MODE_F32SCALE, st), "dequant")

        for _ in range(n):
            quant()
        launches = max(8, min(64, (8 << 30) // touched))
        q_us = _time_back_to_back(quant, launches)
        d_us = _time_back_to_back(dequant, launches)
        algo = 3 * M * N + 4 * (M // 128) * (N // 128)
        rows.append({"shape": [M, N], "algorithmic_MB": algo / 1e6, "quant_us": q_us, "dequant_us": d_us,
                     "quant_hbm_frac": algo / q_us / 1e3 / HBM_PEAK_GBS, "dequant_hbm_frac": algo / d_us / 1e3 / HBM_PEAK_GBS,
                     # what is left of a launch when its bytes are charged at the rate of the largest launch of this sweep
                     "buffers_cycled": n})
        del ws, qs, ss, ys
        torch.cuda.empty_cache()
    best_q = max(r["quant_hbm_frac"] for r in rows)
    best_d = max(r["dequant_hbm_frac"] for r in rows)
    for r in rows:
        r["quant_fixed_us"] = r["quant_us"] - r["algorithmic_MB"] / (best_q * HBM_PEAK_GBS) * 1e3
        r["dequant_fixed_us"] = r["dequant_us"] - r["algorithmic_MB"] / (best_d * HBM_PEAK_GBS) * 1e3
    return {"workload": "one bf16 [M, N] matrix per launch, block-FP8 quant (headline arithmetic) and dequant, launches back to "
                        "back between one pair of events, cold buffers; *_fixed_us = time of a launch beyond its bytes at the "
                        "rate of the best launch of the sweep",
            "empty_launch_us_back_to_back": empty_b2b, "rows": rows}


def bench_fp8_quant_moe(dev, steps, warmup, layers, mode=HEADLINE_FP8_MODE):
    """Block-FP8 quant of every linear weight of a Qwen3-30B-A3B-shaped state dict (48 layers: 128 experts x
    gate/up [768,2048], down [2048,768]; attention q [4096,2048], k/v [512,2048], o [2048,4096]), one grouped launch."""
    import torch

    import slime_amd
    from oracle import c_oracle

    weights, _ = _moe_state_dict(dev, layers)
    plan = slime_amd.Fp8QuantPlan(weights, (128, 128), mode=mode)
    wall_ms, ev_ms, ev_min = _time_launches(plan.run, steps, warmup)
    elements = sum(w.numel() for w in weights)
    algo_bytes = 3 * elements + 4 * plan.total_tiles
    for idx in (0, 2, 385, len(weights) - 1):
        q, s = plan.outputs[idx]
        qo, so = c_oracle.fp8_block_quant(weights[idx].cpu().contiguous(), (128, 128), plan.mode)
        assert torch.equal(q.cpu().view(torch.uint8), qo) and torch.equal(s.cpu().view(torch.int32), so.view(torch.int32))
    out = {"workload": f"Qwen3-30B-A3B-shaped state dict, {layers} layers x (128 experts x gate, up [768,2048], down "
                       f"[2048,768] + q, k, v, o), block-FP8 128x128 (arithmetic mode {mode}), one grouped launch",
           "mode": mode, "tensors": len(weights), "bf16_GB": 2 * elements / 1e9, "kernel_ms": ev_ms, "wall_ms": wall_ms,
           "bf16_GBps": 2 * elements / ev_ms / 1e6, "algo_GBps": algo_bytes / ev_ms / 1e6,
           "hbm_frac": algo_bytes / ev_ms / 1e6 / HBM_PEAK_GBS, "parity_tensors_checked": 4}
    del plan, weights
    torch.cuda.empty_cache()
    return out


def bench_bucket(dev, steps, warmup, layers):
    """The weight-sync drop-in: the Qwen3-30B-A3B-shaped state dict after name conversion - per layer 128 experts
    (gate/up as chunk views of one fc1 weight, down), q/k/v from one fused parameter, o, two norms and the router -
    through BucketConverter, as ONE bucket (launches per sync = 1) and as one bucket per layer."""
    import torch

    from oracle import c_oracle
    from slime_amd import bucket as B

    cfg = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic", "weight_block_size": [128, 128]}
    def make_layer(layer):
        L, hf = f"module.module.decoder.layers.{layer}.", f"model.layers.{layer}."
        fc1 = _gen_bf16((128, 2 * 768, 2048), dev, outliers=True)
        fc2 = _gen_bf16((128, 2048, 768), dev, outliers=True)
        params = [(L + "self_attention.linear_qkv.layer_norm_weight", [(hf + "input_layernorm.weight", _gen_bf16((2048,), dev))]),
                  (L + "self_attention.linear_qkv.weight", [(hf + "self_attn.q_proj.weight", _gen_bf16((4096, 2048), dev)),
                                                          (hf + "self_attn.k_proj.weight", _gen_bf16((512, 2048), dev)),
                                                          (hf + "self_attn.v_proj.weight", _gen_bf16((512, 2048), dev))]),
                  (L + "self_attention.linear_proj.weight", [(hf + "self_attn.o_proj.weight", _gen_bf16((2048, 4096), dev))]),
                  (L + "pre_mlp_layernorm.weight", [(hf + "post_attention_layernorm.weight", _gen_bf16((2048,), dev))]),
                  (L + "mlp.router.weight", [(hf + "mlp.gate.weight", _gen_bf16((128, 2048), dev))])]
        for e in range(128):
            gate, up = fc1[e].chunk(2, dim=0)
            params.append((L + f"mlp.experts.linear_fc1.weight{e}",
                           [(hf + f"mlp.experts.{e}.gate_proj.weight", gate), (hf + f"mlp.experts.{e}.up_proj.weight", up)]))
            params.append((L + f"mlp.experts.linear_fc2.weight{e}", [(hf + f"mlp.experts.{e}.down_proj.weight", fc2[e])]))
        return params

    per_layer = [make_layer(layer) for layer in range(layers)]
    whole = [p for params in per_layer for p in params]
    n_tensors = sum(len(cv) for _, cv in whole)
    quantised = [(n, t) for _, cv in whole for n, t in cv if n.endswith("proj.weight")]
    elements = sum(t.numel() for _, t in quantised)
    algo_bytes = 3 * elements + 4 * sum((-(-t.shape[0] // 128)) * (-(-t.shape[1] // 128)) for _, t in quantised)
    conv = B.BucketConverter(None, cfg)
    state = {}

    def one_bucket():
        state["out"] = None                       # the previous sync's buffer goes back to the allocator first
        state["out"] = conv.convert(whole, bucket_id="all")

    def per_layer_buckets():
        state["out"] = None
        state["out"] = [conv.convert(params, bucket_id=i) for i, params in enumerate(per_layer)]

    t0 = time.perf_counter()
    one_bucket()
    torch.cuda.synchronize()
    first_ms = (time.perf_counter() - t0) * 1e3
    wall1, _, _ = _time_launches(one_bucket, steps, warmup)
    # the call pattern of a sharded model: every sync presents the same names and shapes in freshly allocated tensors.
    # A second copy of the state dict at other addresses, alternated with the first: every sync is a miss.
    other = [p for layer in range(layers) for p in make_layer(layer)]
    sets = [whole, other]
    state["k"] = 0

    def one_bucket_moved():
        state["out"] = None
        state["k"] ^= 1
        state["out"] = conv.convert(sets[state["k"]], bucket_id="all")

    def one_bucket_no_id():                      # the layout found by names, shapes, dtypes and strides instead of an id
        state["out"] = None
        state["out"] = conv.convert(whole)

    wall_noid, _, _ = _time_launches(one_bucket_no_id, steps, warmup)
    resolves0 = conv.resolves
    wall_moved, _, _ = _time_launches(one_bucket_moved, steps, warmup)
    moved_resolves = conv.resolves - resolves0
    named = dict(state["out"].reconstruct_tensors())
    src = dict((n, t) for _, cv in sets[state["k"]] for n, t in cv)
    for n in (quantised[0][0], quantised[-1][0]):
        qo, so = c_oracle.fp8_block_quant(src[n].cpu().contiguous(), (128, 128), 1)
        assert torch.equal(named[n].cpu().view(torch.uint8), qo), "moved bucket: FP8 parity failure"
        assert torch.equal(named[n.replace(".weight", ".weight_scale_inv")].cpu().view(torch.int32), so.view(torch.int32))
    assert moved_resolves == steps + warmup and conv.plan_builds == 2       # one layout per key: by id, by identity
    del named, src, other, sets
    state["out"] = None
    torch.cuda.empty_cache()
    one_bucket()                                  # back on the first set for the kernel timing below
    conv.time_kernels = True
    for _ in range(steps):
        one_bucket()
    torch.cuda.synchronize()
    ev1 = conv.kernel_ms() / steps
    launches1 = state["out"].launches
    named = dict(state["out"].reconstruct_tensors())
    for n, t in (quantised[0], quantised[5], quantised[-1]):
        qo, so = c_oracle.fp8_block_quant(t.cpu().contiguous(), (128, 128), 1)
        assert torch.equal(named[n].cpu().view(torch.uint8), qo)
        assert torch.equal(named[n.replace(".weight", ".weight_scale_inv")].cpu().view(torch.int32), so.view(torch.int32))
    assert torch.equal(named["model.layers.0.mlp.gate.weight"], whole[4][1][0][1])
    del named
    conv.time_kernels = False
    wallL, _, _ = _time_launches(per_layer_buckets, steps, warmup)
    conv.time_kernels = True
    for _ in range(steps):
        per_layer_buckets()
    torch.cuda.synchronize()
    evL = conv.kernel_ms() / steps
    launchesL = sum(b.launches for b in state["out"])
    state["out"] = None
    # the INT4 weight sync of the same state dict: experts to compressed-tensors INT4 (symmetric, group 128, the
    # converter's default ignore rules), everything else copied through; one bucket per layer
    cfg4 = {"quant_method": "compressed-tensors",
            "config_groups": {"group_0": {"weights": {"group_size": 128, "symmetric": True, "num_bits": 4}}},
            "ignore": ["re:.*lm_head.*", "re:.*norm.*", "re:.*embed.*", "re:.*self_attn.*", "re:.*shared_experts.*",
                       "re:.*mlp\\.(gate|up|gate_up|down)_proj.*", "re:.*mlp\\.gate\\.*"]}
    conv4 = B.BucketConverter(None, cfg4)

    def int4_per_layer():
        state["out"] = None
        state["out"] = [conv4.convert(params, bucket_id=i) for i, params in enumerate(per_layer)]

    wall4, _, _ = _time_launches(int4_per_layer, steps, warmup)
    conv4.time_kernels = True
    for _ in range(steps):
        int4_per_layer()
    torch.cuda.synchronize()
    ev4 = conv4.kernel_ms() / steps
    launches4 = sum(b.launches for b in state["out"])
    named4 = dict(state["out"][0].reconstruct_tensors())
    n0, t0_ = quantised[4]                                   # an expert projection of layer 0
    assert ".experts." in n0
    po, so, _ = c_oracle.int4_pack_layer(t0_.cpu().contiguous(), 128, True)
    assert torch.equal(named4[n0.replace(".weight", ".weight_packed")].cpu(), po)
    assert torch.equal(named4[n0.replace(".weight", ".weight_scale")].cpu().view(torch.int16), so.view(torch.int16))
    expert_el = sum(t.numel() for n, t in quantised if ".experts." in n)
    passed = sum(t.numel() * t.element_size() for _, cv in whole for n, t in cv if ".experts." not in n)
    algo4 = int(expert_el * 2.515625) + 2 * passed
    del named4
    # the same conversion as ONE bucket: one launch instead of 48, so one start-up and one tail instead of 48
    conv4.time_kernels = False

    def int4_one_bucket():
        state["out"] = None
        state["out"] = conv4.convert(whole, bucket_id="all")

    wall4a, _, _ = _time_launches(int4_one_bucket, steps, warmup)
    conv4.time_kernels = True
    for _ in range(steps):
        int4_one_bucket()
    torch.cuda.synchronize()
    ev4a = conv4.kernel_ms() / steps
    launches4a = state["out"].launches
    del conv4
    state["out"] = None
    # the loop this replaces, on this build's own per-tensor kernels (so the difference is launches and copies, not
    # arithmetic): quantize_params per Megatron parameter, then the flatten copy; two layers, scaled to all of them
    sample = per_layer[:2]

    def loop_and_flatten():
        state["out"] = None
        state["out"] = [B.flatten_named_tensors(B.per_param_loop(None, params, cfg)) for params in sample]

    wallP, _, _ = _time_launches(loop_and_flatten, 5, 3)       # three warm-up passes: the allocator has every block the loop needs
    state["out"] = None
    out = {"workload": f"Qwen3-30B-A3B-shaped state dict after name conversion, {layers} layers, {n_tensors} tensors "
                       f"({len(quantised)} quantised to block-FP8 with the weight-sync arithmetic, the rest copied), written "
                       "into the one uint8 buffer + metadata a FlattenedTensorBucket consumer reads; fresh output buffer per sync",
           "tensors": n_tensors, "bf16_GB": 2 * elements / 1e9,
           "one_bucket": {"launches_per_sync": launches1, "ms_per_sync_kernels": ev1, "ms_per_sync_wall": wall1,
                          "ms_per_sync_wall_without_bucket_id": wall_noid,
                          "ms_per_sync_wall_inputs_reallocated_every_sync": wall_moved,
                          "reallocated_note": "two copies of the state dict at different addresses alternate, so every sync "
                                              "finds its inputs moved: one upload of 18 768 addresses and one resolve launch "
                                              "over the per-item template, then the same conversion launch",
                          "first_call_ms_layout_build": first_ms, "hbm_frac": algo_bytes / ev1 / 1e6 / HBM_PEAK_GBS,
                          "bf16_GBps": 2 * elements / ev1 / 1e6},
           "bucket_per_layer": {"launches_per_sync": launchesL, "ms_per_sync_kernels": evL, "ms_per_sync_wall": wallL,
                                "hbm_frac": algo_bytes / evL / 1e6 / HBM_PEAK_GBS, "bf16_GBps": 2 * elements / evL / 1e6},
           "int4_bucket_per_layer": {"what": "the same state dict through the compressed-tensors INT4 branch: 18 432 expert "
                                             "weights packed (sym, group 128), attention / norms / router copied through",
                                     "launches_per_sync": launches4, "ms_per_sync_kernels": ev4, "ms_per_sync_wall": wall4,
                                     "hbm_frac": algo4 / ev4 / 1e6 / HBM_PEAK_GBS, "bf16_GBps": 2 * expert_el / ev4 / 1e6},
           "int4_one_bucket": {"what": "the INT4 branch with the whole state dict as one bucket",
                               "launches_per_sync": launches4a, "ms_per_sync_kernels": ev4a, "ms_per_sync_wall": wall4a,
                               "hbm_frac": algo4 / ev4a / 1e6 / HBM_PEAK_GBS, "bf16_GBps": 2 * expert_el / ev4a / 1e6},
           "per_parameter_loop_then_flatten": {
               "what": "quantize_params once per Megatron parameter (one launch each) followed by the flatten "
                       "copy into one buffer, per layer bucket - the shape of the reference's loop, on this build's kernels",
               "ms_per_sync_wall": wallP * layers / len(sample), "measured_on_layers": len(sample),
               "quantiser_launches_per_sync": 258 * layers},
           "table_builds": conv.plan_builds, "parity_tensors_checked": 3}
    del state, conv, whole, per_layer, quantised
    torch.cuda.empty_cache()
    return out


def bench_bucket_off_lines(dev, steps, warmup, layers=6):
    """A DeepSeek-V3-shaped (MLA) FP8 weight-sync bucket: kv_a_proj_with_mqa [576, 7168] has 280 tiles, so its 1120 bytes
    of scales leave every tensor packed after it 96 bytes off the 128-byte lines of the flat buffer.  Those tensors take the
    converter's second launch (plain stores); the record says what the bucket costs and checks a tensor from each launch."""
    import torch

    from oracle import c_oracle
    from slime_amd import bucket as B

    cfg = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic", "weight_block_size": [128, 128]}
    params = []
    for layer in range(layers):
        L, hf = f"module.module.decoder.layers.{layer}.", f"model.layers.{layer}."
        params += [(L + "self_attention.linear_q_down_proj.weight", [(hf + "self_attn.q_a_proj.weight", _gen_bf16((1536, 7168), dev))]),
                   (L + "self_attention.linear_q_up_proj.weight", [(hf + "self_attn.q_b_proj.weight", _gen_bf16((24576, 1536), dev))]),
                   (L + "self_attention.linear_kv_down_proj.weight", [(hf + "self_attn.kv_a_proj_with_mqa.weight", _gen_bf16((576, 7168), dev))]),
                   (L + "self_attention.linear_kv_up_proj.weight", [(hf + "self_attn.kv_b_proj.weight", _gen_bf16((32768, 512), dev))]),
                   (L + "self_attention.linear_proj.weight", [(hf + "self_attn.o_proj.weight", _gen_bf16((7168, 16384), dev))])]
        for e in range(16):
            params.append((L + f"mlp.experts.linear_fc2.weight{e}",
                           [(hf + f"mlp.experts.{e}.down_proj.weight", _gen_bf16((7168, 2048), dev, outliers=True))]))
    tensors = [(n, t) for _, cv in params for n, t in cv]
    elements = sum(t.numel() for _, t in tensors)
    algo = 3 * elements + 4 * sum((-(-t.shape[0] // 128)) * (-(-t.shape[1] // 128)) for _, t in tensors)
    conv = B.BucketConverter(None, cfg)
    state = {}

    def run():
        state["out"] = None
        state["out"] = conv.convert(params, bucket_id="mla")

    wall, _, _ = _time_launches(run, steps, warmup)
    conv.time_kernels = True
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    ev = conv.kernel_ms() / steps
    out = state["out"]
    off = sum(1 for m in out.metadata if m.dtype == torch.float8_e4m3fn and m.start_idx % 64)
    named = dict(out.reconstruct_tensors())
    for n, t in (tensors[0], tensors[3], tensors[-1]):                 # before and after the tensor that shifts the rest
        qo, so = c_oracle.fp8_block_quant(t.cpu().contiguous(), (128, 128), 1)
        assert torch.equal(named[n].cpu().view(torch.uint8), qo), f"off-line bucket: parity failure on {n}"
        assert torch.equal(named[n.replace(".weight", ".weight_scale_inv")].cpu().view(torch.int32), so.view(torch.int32))
    return {"workload": f"{layers} layers x (q_a [1536,7168], q_b [24576,1536], kv_a [576,7168], kv_b [32768,512], o [7168,16384], 16 experts' "
                        "down [7168,2048]) bf16 -> block-FP8 through BucketConverter, packed back to back",
            "tensors": len(tensors), "tensors_off_the_lines": off, "launches_per_sync": out.launches, "ms_per_sync_kernels": ev,
            "ms_per_sync_wall": wall, "hbm_frac": algo / ev / 1e6 / HBM_PEAK_GBS, "bf16_GBps": 2 * elements / ev / 1e6,
            "parity_tensors_checked": 3}


def bench_grouped_experts(dev, steps, warmup, experts=128):
    """The stacked expert weights of one MoE layer's grouped linears (fc1 = gate+up [1536, 2048], fc2 [2048, 768]) as the
    FP8-aligned MoE forward quantises them on every step: one launch per grouped linear against the loop it replaces."""
    import torch

    import slime_amd

    fc1 = [_gen_bf16((1536, 2048), dev, outliers=True) for _ in range(experts)]
    fc2 = [_gen_bf16((2048, 768), dev, outliers=True) for _ in range(experts)]

    def one_launch():
        slime_amd.quantize_grouped_weights(fc1, (128, 128))
        slime_amd.quantize_grouped_weights(fc2, (128, 128))

    def loop():
        for ws, shape in ((fc1, (1536, 2048)), (fc2, (2048, 768))):
            q = torch.empty((experts, *shape), dtype=torch.float8_e4m3fn, device=dev)
            s = torch.empty((experts, shape[0] // 128, shape[1] // 128), dtype=torch.float32, device=dev)
            for e, w in enumerate(ws):
                qe, se = slime_amd.blockwise_cast_to_fp8_triton(w, (128, 128))
                q[e].copy_(qe)
                s[e].copy_(se)

    wall1, ev1, _ = _time_launches(one_launch, steps, warmup)
    wall2, ev2, _ = _time_launches(loop, max(steps // 4, 2), 1)
    q, s = slime_amd.quantize_grouped_weights(fc1, (128, 128))
    qe, se = slime_amd.blockwise_cast_to_fp8_triton(fc1[7], (128, 128))
    assert torch.equal(q[7].view(torch.uint8), qe.view(torch.uint8)) and torch.equal(s[7], se)
    el = experts * (1536 * 2048 + 2048 * 768)
    algo = 3 * el + 4 * el // 16384
    return {"workload": f"{experts} experts x (fc1 [1536,2048], fc2 [2048,768]) bf16 -> stacked e4m3 [E,N,K] + fp32 scales, "
                        "one launch per grouped linear (table cached on the weight addresses)",
            "ms": ev1, "wall_ms": wall1, "hbm_frac": algo / ev1 / 1e6 / HBM_PEAK_GBS,
            "per_expert_loop_ms": ev2, "per_expert_loop_wall_ms": wall2, "launches": 2, "loop_launches": 6 * experts}


def bench_int4_pack(dev, steps, warmup, layers):
    import torch

    import slime_amd
    from oracle import c_oracle

    _, weights = _moe_state_dict(dev, layers)
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
    of `layers` Qwen3-30B-A3B layers, every expert its own tensor, one launch per step."""
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
        # every expert its own weight (views of the layer's tensors), all of them through one launch
        per_expert = []
        for t in tensors:
            r = t.shape[0] // 128
            per_expert += [t[e * r:(e + 1) * r] for e in range(128)]
        ste_plan = slime_amd.Int4StePlan(per_expert, 128)

        def run():
            outs[0] = ste_plan.run()

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
            r = tensors[idx].shape[0] // 128
            got = torch.cat([outs[0][idx * 128 + e] for e in range(-(-1024 // r))])[:1024]
        assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))
    launches = 1
    out = {"workload": f"Qwen3-30B-A3B experts, {layers} layers x (gate, up [128x768,2048], down [128x2048,768]), "
                       + ("INT4 group 128 -> bf16" if which == "int4deq" else "INT4 QAT quantise-dequantise forward")
                       + f", {len(tensors) * 128} expert tensors in one launch"
,
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

    plan = delta.XorDiffPlan(news, olds)             # per-chunk descriptors built once; two launches per run

    def run():
        plan.run(update_snapshot=True)

    wall_ms, ev_ms, ev_min = _time_launches(run, steps, warmup)
    news[5][:4096] ^= 3                                # the timed form, checked too: a fresh difference in one tensor
    check_new, check_old = news[5].cpu().numpy(), olds[5].cpu().numpy().copy()
    diffs, results = plan.run(update_snapshot=True)
    torch.cuda.synchronize()
    want, changed = delta_ref.xor_delta_ref(check_new, check_old)
    assert np.array_equal(diffs[5].cpu().numpy(), want) and np.array_equal(olds[5].cpu().numpy(), check_new)
    assert results[5].tolist() == [changed, int(delta_ref.adler32_ref(check_new), 16)] and changed == 4096
    nbytes = sum(nw.numel() for nw in news)
    xxh3 = _bench_xxh3(news, steps, warmup)
    fused = _bench_delta_with_digest(news, olds, steps, warmup)
    out = {"xxh3_128": xxh3, "with_xxh3_digest": fused,
           "workload": "Qwen3-4B-shaped state dict (252 bf16 tensors, 7.27 GB) against its snapshot in HBM: xor diff, "
                       "changed-byte count, adler32, snapshot update; two launches for the whole bucket",
           "tensors": len(news), "weight_GB": nbytes / 1e9, "kernel_ms": ev_ms, "wall_ms": wall_ms,
           "weight_GBps": nbytes / ev_ms / 1e6, "algo_GBps": 4 * nbytes / ev_ms / 1e6,
           "hbm_frac": 4 * nbytes / ev_ms / 1e6 / HBM_PEAK_GBS, "parity_tensors_checked": 2}
    del news, olds, plan
    torch.cuda.empty_cache()
    return out


def _bench_delta_with_digest(news, olds, steps, warmup):
    """The delta pass with the default digest riding on it: the bytes the diff reads also feed XXH3's block sums, one more
    launch walks them - three launches for diff, counts, adler32, snapshot update and xxh3-128 of the whole bucket."""
    import torch

    from slime_amd import delta

    plan = delta.XorDiffPlan(news, olds, xxh3=True)
    wall_ms, ev_ms, _ = _time_launches(lambda: plan.run(update_snapshot=True), steps, warmup)
    news[2][100:200] ^= 5
    plan.run(update_snapshot=True)
    got = plan.hexdigests()
    assert got[2] == delta.xxh3_128(news[2]) and all(g is None for i, g in enumerate(got) if i != 2)
    # timed runs above ran on an unchanged bucket (no digest walk); time the walk with every tensor changed
    torch.cuda.synchronize()
    t = []
    for _ in range(max(steps // 2, 3)):
        for old in olds:
            old[0] ^= 1                                     # one byte per tensor differs again: every digest is walked
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        plan.run(update_snapshot=True)
        e1.record()
        torch.cuda.synchronize()
        t.append(e0.elapsed_time(e1))
    assert plan.results[:, 0].tolist() == [1] * len(news) and plan.hexdigests()[4] == delta.xxh3_128(news[4])
    nbytes = sum(nw.numel() for nw in news)
    ms = sum(t) / len(t)
    return {"workload": "the same pass with the xxh3-128 digest of every tensor computed from the bytes the diff reads "
                        "(64 bytes of block sums per KiB written by the diff kernel, then the per-tensor walk): three launches",
            "ms_all_tensors_changed": ms, "ms_no_tensor_changed": ev_ms, "weight_GBps": nbytes / ms / 1e6,
            "hbm_frac_of_diff_kernel_when_unchanged": (4 + 1 / 16) * nbytes / ev_ms / 1e6 / HBM_PEAK_GBS}


def _bench_xxh3(news, steps, warmup):
    """The digest the reference's delta publisher attaches by default, over the same state dict: two launches (block sums
    at memory speed, then one scramble chain per tensor), against the xxhash package on the host for one tensor."""
    import torch

    from slime_amd import delta

    plan = delta.Xxh3Plan(news)             # table, workspace and digest buffer set up once

    wall_ms, ev_ms, _ = _time_launches(plan.run, max(steps // 2, 3), 2)
    assert plan.hexdigests()[4] == delta.xxh3_128(news[4])
    nbytes = sum(nw.numel() for nw in news)
    rec = {"workload": "xxh3-128 of every tensor of the same state dict (read once; 64 bytes of block sums per KiB, then a "
                       "sequential chain of 48 640 blocks for the largest tensor)",
           "ms": ev_ms, "wall_ms": wall_ms, "weight_GBps": nbytes / ev_ms / 1e6, "hbm_frac": (nbytes * 17 / 16) / ev_ms / 1e6 / HBM_PEAK_GBS}
    try:
        import xxhash

        got = delta.xxh3_128(news[4])
        host = news[4].cpu().numpy().tobytes()
        t0 = time.perf_counter()
        want = xxhash.xxh3_128(host).hexdigest()
        rec["host_one_thread_GBps"] = len(host) / (time.perf_counter() - t0) / 1e9
        assert got == want
        rec["parity"] = "digest of a 49.8 MB tensor equals xxhash.xxh3_128 on the host"
    except ImportError:
        rec["parity"] = "xxhash package not installed: not checked in this run"
    return rec


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
             ("int4_fake_quant_asym", lambda: slime_amd.fake_int4_quant_cuda(w, (1, 128), False), 4 * el + 4 * el // 128),
             # FP8-aligned weight: quantise + expand in one pass (4 bytes per element), and the two kernels it replaces
             ("fp8_aligned_weight", lambda: slime_amd.fp8_aligned_weight(w), 4 * el),
             ("fp8_quant_then_dequant", lambda: slime_amd.block_quant_dequant(
                 *slime_amd.blockwise_cast_to_fp8_triton(w, (128, 128)), [128, 128], torch.bfloat16), 6 * el))
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
    y = slime_amd.fp8_aligned_weight(w)
    qo, so = c_oracle.fp8_block_quant(head, (128, 128), 1)
    assert torch.equal(y[:512].cpu().view(torch.int16), c_oracle.fp8_block_dequant(qo, so, 128, 0).view(torch.int16))
    out["workload"] = ("one bf16 [151936, 2560] tensor (778 MB); algorithmic bytes per element: channel 3, tensor 5 (two "
                       "reads), fake INT4 4, FP8-aligned weight 4 (the quantiser followed by the dequantiser: 6); parity "
                       "checked on the first 512 rows")
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

    import wq_testlib
    from slime_amd import _lib

    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 256)
    dst = torch.empty_like(src)

    def run():
        _lib.check(wq_testlib.load().wq_copy_bytes(src.data_ptr(), dst.data_ptr(), nbytes, _lib.stream_ptr(dev)), "copy")

    wall_ms, ev_ms, ev_min = _time_launches(run, steps, warmup)
    assert torch.equal(src[:1 << 20], dst[:1 << 20]) and torch.equal(src[-(1 << 20):], dst[-(1 << 20):])
    rec = {"workload": "copy_kernel 4 GiB", "bytes_read": nbytes, "bytes_written": nbytes, "kernel_ms": ev_ms,
           "kernel_ms_min": ev_min, "GBps_read_plus_write": 2 * nbytes / ev_ms / 1e6,
           "hbm_frac": 2 * nbytes / ev_ms / 1e6 / HBM_PEAK_GBS}
    # the same for the quantisers' read:write mixes: compute-free 2:1 and 4:1 streams over the same 4 GiB of input
    for ratio in (2, 4):
        n_out = nbytes // ratio

        def fold():
            _lib.check(wq_testlib.load().wq_stream_fold_bytes(src.data_ptr(), dst.data_ptr(), n_out, ratio, _lib.stream_ptr(dev)), "fold")

        _, f_ms, f_min = _time_launches(fold, steps, warmup)
        piece = {2: 16384, 4: 8192}[ratio]                   # bytes of output per work item
        pieces = src[:ratio * piece].view(ratio, piece)
        want = pieces[0].clone()
        for r in range(1, ratio):
            want ^= pieces[r]
        assert torch.equal(dst[:piece], want)
        rec[f"compute_free_{ratio}_to_1"] = {"bytes_read": nbytes, "bytes_written": n_out, "kernel_ms": f_ms, "kernel_ms_min": f_min,
                                              "hbm_frac": (nbytes + n_out) / f_ms / 1e6 / HBM_PEAK_GBS}
    # and for the dequantisers' mixes: compute-free 1:2 and 1:4 streams (1 GiB read, 2 / 4 GiB written)
    n_in = nbytes // 4
    for ratio in (2, 4):

        def expand():
            _lib.check(wq_testlib.load().wq_stream_expand_bytes(src.data_ptr(), dst.data_ptr(), n_in, ratio, _lib.stream_ptr(dev)), "expand")

        _, x_ms, x_min = _time_launches(expand, steps, warmup)
        head = dst[:ratio * 4096].view(torch.int32).view(ratio, 1024)
        first = src[:4096].view(torch.int32)
        assert all(torch.equal(head[w], first + w) for w in range(ratio))
        rec[f"compute_free_1_to_{ratio}"] = {"bytes_read": n_in, "bytes_written": ratio * n_in, "kernel_ms": x_ms, "kernel_ms_min": x_min,
                                              "hbm_frac": (1 + ratio) * n_in / x_ms / 1e6 / HBM_PEAK_GBS}
    return rec


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


def _cpu_gen(shape, seed, outliers=True):
    import torch

    g = torch.Generator().manual_seed(seed)
    w = torch.randn(shape, generator=g) * 0.02
    if outliers:
        w[torch.rand(shape, generator=g) < 1e-3] *= 20
    return w.to(torch.bfloat16)


def _cpu_rate(fn, nbytes, budget_s, max_reps=500):
    """Runs fn (one pass over the sample) until the time budget is used.  -> (GB/s of bf16, passes, seconds)."""
    fn()                                       # warm the allocator and the thread pool
    reps, t0 = 0, time.perf_counter()
    while True:
        fn()
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or reps >= max_reps:
            break
    return nbytes * reps / dt / 1e9, reps, dt


def cpu_baselines(budget_s: float, north_star_bytes):
    """The CPU restatements of the reference's torch path (oracle/torch_ref.py: the same op sequences as
    convert_hf_to_fp8.block_fp8, convert_hf_to_int4_direct.pack_layer and fp8_cast_bf16.weight_dequant), timed on
    this box's host cores on bounded samples of the benchmark's own tensor shapes.
    -> (the `cpu_baseline` object of the headline step, {leg: record})."""
    import torch

    from oracle import torch_ref

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    cores = torch.get_num_threads()
    unit = "GB/s of bf16 weights"
    legs = {}

    # Qwen3-30B-A3B: 8 experts of one layer (24 tensors) + the layer's q, k, v, o
    experts = [_cpu_gen(sh, 10 + i) for i, sh in enumerate([(768, 2048), (768, 2048), (2048, 768)] * 8)]
    attn = [_cpu_gen(sh, 50 + i, False) for i, sh in enumerate([(4096, 2048), (512, 2048), (512, 2048), (2048, 4096)])]
    nb = sum(2 * w.numel() for w in experts + attn)
    rate_fp8, reps, dt = _cpu_rate(lambda: [torch_ref.block_fp8_ref(w, (128, 128)) for w in experts + attn], nb, budget_s * 0.3)
    legs["fp8_block_quant"] = {"value": rate_fp8, "unit": unit, "cores": cores, "kind": "port",
                               "sample": f"8 experts (gate, up, down) + q, k, v, o of one Qwen3-30B-A3B-shaped layer "
                                         f"({nb / 1e6:.0f} MB bf16) x {reps} passes in {dt:.1f} s, torch CPU restatement of block_fp8"}
    nb = sum(2 * w.numel() for w in experts)
    rate_int4, reps, dt = _cpu_rate(lambda: [torch_ref.pack_layer_ref(w, 128, True) for w in experts], nb, budget_s * 0.3)
    legs["int4_group_quant_pack"] = {"value": rate_int4, "unit": unit, "cores": cores, "kind": "port",
                                     "sample": f"8 experts (gate, up, down) of one Qwen3-30B-A3B-shaped layer ({nb / 1e6:.0f} MB "
                                               f"bf16) x {reps} passes in {dt:.1f} s, torch CPU restatement of the "
                                               "fake_int4_quant_cuda kernel + pack_layer"}
    del experts, attn

    # DeepSeek-V3: 8 experts (24 tensors) of e4m3 codes + scales -> bf16
    g = torch.Generator().manual_seed(7)
    xs, ss = [], []
    for sh in [(2048, 7168), (2048, 7168), (7168, 2048)] * 8:
        c = torch.randint(0, 254, sh, generator=g, dtype=torch.int32)
        xs.append((c + (c >= 0x7F).int()).to(torch.uint8).view(torch.float8_e4m3fn))
        ss.append(torch.exp(torch.empty(sh[0] // 128, sh[1] // 128).uniform_(-9.21034, -2.302585, generator=g)))
    nb = sum(2 * x.numel() for x in xs)
    rate, reps, dt = _cpu_rate(lambda: [torch_ref.weight_dequant_ref(x, sc) for x, sc in zip(xs, ss)], nb, budget_s * 0.2)
    legs["fp8_block_dequant"] = {"value": rate, "unit": "GB/s of bf16 weights produced", "cores": cores, "kind": "port",
                                 "sample": f"8 experts (gate, up, down) of the DeepSeek-V3-shaped layer ({nb / 1e6:.0f} MB bf16 "
                                           f"out) x {reps} passes in {dt:.1f} s, torch CPU restatement of weight_dequant"}
    del xs, ss

    # the [4096, 4096] matrix in full: quant, then dequant of its own output
    w = _cpu_gen((4096, 4096), 0)

    def cfg1():
        q, sc = torch_ref.block_fp8_ref(w, (128, 128))
        torch_ref.weight_dequant_ref(q, sc)

    rate, reps, dt = _cpu_rate(cfg1, 2 * w.numel(), budget_s * 0.2)
    legs["cfg1_roundtrip"] = {"value": rate, "unit": "GB/s of bf16 weights through quant + dequant", "cores": cores,
                              "kind": "port", "sample": f"the whole [4096,4096] matrix x {reps} round trips in {dt:.1f} s, "
                                                        "torch CPU restatement of block_fp8 + weight_dequant"}

    b_fp8, b_int4 = north_star_bytes
    mixed = (b_fp8 + b_int4) / (b_fp8 / rate_fp8 + b_int4 / rate_int4)
    head = {"value": mixed, "unit": unit, "cores": cores, "kind": "port",
            "sample": "the step's mix of block-FP8 and INT4 work at the CPU rates measured on 8 experts + q, k, v, o of one "
                      f"layer: FP8 {rate_fp8:.2f} GB/s, INT4 {rate_int4:.2f} GB/s (records under cpu_baseline_legs); torch CPU "
                      "op-for-op restatements of block_fp8 and fake_int4_quant_cuda + pack_layer"}
    return head, legs


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--cpu-seconds", type=float, default=24.0, help="time budget of the CPU baseline samples (all legs)")
    ap.add_argument("--int4-layers", type=int, default=48, help="layers of Qwen3-30B-A3B experts in the INT4 extra")
    ap.add_argument("--dequant-experts", type=int, default=256)
    ap.add_argument("--no-extras", action="store_true", help="headline step only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--only", choices=["fp8", "cfg1", "bucket", "fp8moe", "int4", "dequant", "int4deq", "ste", "delta", "forms", "experts", "copy", "stream", "sizes", "mla", "hashes"], default=None,
                    help="run just one of the other legs and print its record: a kernel for profiling, the plain copy "
                         "kernel that hardware counters are calibrated against, or the host-resident streaming run "
                         "(64 x 1 GiB buckets, PCIe-bound)")
    ap.add_argument("--fp8-mode", type=int, default=HEADLINE_FP8_MODE, choices=[0, 1, 2],
                    help="arithmetic of `--only fp8moe`: 0 block_fp8 on CPU tensors (the headline), 1 weight-sync cast, 2 block_fp8 on GPU tensors")
    ap.add_argument("--stream-buckets", type=int, default=64)
    ap.add_argument("--stream-bucket-mib", type=int, default=1024)
    ap.add_argument("--stream-no-download", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures ONE GPU: the path has no cross-GPU exchange and this build has no multi-GPU "
              "launcher; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.only == "hashes":       # what the profile summaries record as kernel_source_sha256
        print(json.dumps({k: kernel_source_hash(*v) for k, v in KERNEL_SOURCES.items()}))
        return

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.manual_seed(0)

    if args.only == "fp8":
        print(json.dumps(bench_fp8_quant(dev, args.steps, args.warmup)))
        return
    if args.only == "cfg1":
        print(json.dumps(bench_cfg1(dev, args.steps, args.warmup)))
        return
    if args.only == "bucket":
        print(json.dumps(bench_bucket(dev, args.steps, args.warmup, args.int4_layers)))
        return
    if args.only == "fp8moe":
        print(json.dumps(bench_fp8_quant_moe(dev, args.steps, args.warmup, args.int4_layers, args.fp8_mode)))
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
    if args.only == "experts":
        print(json.dumps(bench_grouped_experts(dev, args.steps, args.warmup)))
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
    if args.only == "mla":
        print(json.dumps(bench_bucket_off_lines(dev, args.steps, args.warmup)))
        return
    if args.only == "sizes":
        print(json.dumps(bench_launch_sizes(dev)))
        return
    if args.only == "stream":
        print(json.dumps(bench_stream(dev, args.stream_buckets, args.stream_bucket_mib << 20,
                                      not args.stream_no_download)))
        return

    r = bench_north_star(dev, args.steps, args.warmup, args.int4_layers)
    kernels = {}
    for key, name, profile, src in (("fp8", "fp8_block_quant_kernel<TORCH, per-tile descriptors>",
                                     "fp8_block_quant_qwen3_30b_a3b_state_dict.txt", "fp8_block_quant"),
                                    ("int4", "int4_pack_kernel<128, per-item descriptors> (one call = ceil(items / 2^18) dispatches "
                                             "over consecutive parts of the item table; kernel_ms is the call)",
                                     "int4_pack_qwen3_30b_a3b_experts.txt", "int4_pack")):
        k = r[key]
        achieved = k["algo_bytes"] / k["kernel_ms"] / 1e6      # GB/s
        traffic, note = _traffic_from_profile(profile, src)
        kernels[key] = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "traffic_source": note, "kernel": name,
                        "kernel_ms": k["kernel_ms"], "kernel_ms_min": k["kernel_ms_min"],
                        "algorithmic_bytes_per_launch": k["algo_bytes"]}
    lower = min(kernels.values(), key=lambda v: v["frac"])
    line = {
        "metric": "GB/s of bf16 weights quantized (FP8 & INT4) + % of HBM peak, 1x MI355X",
        "value": r["bf16_bytes"] / r["wall_ms"] / 1e6,
        "unit": "GB/s of bf16 weights",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": r["wall_ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"Qwen3-30B-A3B-shaped bf16 state dict ({r['layers']} layers x (128 experts x gate, up "
                               "[768,2048], down [2048,768] + q, k, v, o), N(0, 0.02) with rare x20 outliers), resident in "
                               f"HBM: block-FP8 128x128 quant of all {r['tensors_fp8']} linear weights (block_fp8 arithmetic "
                               f"as torch evaluates it on CPU tensors), then INT4 sym group-128 pack of the {r['tensors_int4']} "
                               "expert weights; one call of the library each (the INT4 call is 14 dispatches of one kernel)",
                   "fp8_mode": r["fp8"]["mode"],
                   "fp8_mode_meaning": "WQ_FP8_MODE_TORCH (0): amax clamped at bf16(1e-12), scale = f32(amax) / 448, q = f32(x) / scale, "
                                       "both IEEE divisions - tools/convert_hf_to_fp8.py:41-75 on CPU tensors, what cpu_baseline computes",
                   "library_calls_per_step": 2, "bf16_GB_fp8": 2 * r["fp8"]["elements"] / 1e9,
                   "bf16_GB_int4": 2 * r["int4"]["elements"] / 1e9, "fp8_blocks": r["fp8"]["blocks"],
                   "parity_tensors_checked": r["parity_tensors_checked"]},
        "pct_hbm_peak": 100.0 * lower["frac"],
        "roofline": lower,
        "roofline_kernels": kernels,
        "fp8_arithmetic_modes": r["fp8_modes"],
    }
    if not args.no_extras:
        extras = {"fp8_block_quant_qwen3_4b": bench_fp8_quant(dev, args.steps, args.warmup),
                  "cfg1_matrix_roundtrip": bench_cfg1(dev, args.steps, args.warmup)}
        if args.dequant_experts > 0:
            extras["fp8_block_dequant"] = bench_fp8_dequant(dev, args.steps, args.warmup, args.dequant_experts)
        if args.int4_layers > 0:
            extras["int4_dequant"] = bench_int4_inverse(dev, args.steps, args.warmup, min(args.int4_layers, 8), "int4deq")
            extras["int4_qat_forward"] = bench_int4_inverse(dev, args.steps, args.warmup, min(args.int4_layers, 8), "ste")
        if args.int4_layers > 0:
            extras["weight_sync_bucket"] = bench_bucket(dev, args.steps, args.warmup, args.int4_layers)
        extras["delta_xor"] = bench_delta(dev, args.steps, args.warmup)
        extras["single_tensor_forms"] = bench_single_tensor_forms(dev, args.steps, args.warmup)
        extras["weight_sync_bucket_off_lines"] = bench_bucket_off_lines(dev, args.steps, args.warmup)
        extras["grouped_expert_weights"] = bench_grouped_experts(dev, args.steps, args.warmup)
        extras["launch_size_curve"] = bench_launch_sizes(dev)
        # config 5's streaming leg: host-resident weights, PCIe-bound by construction (never part of `value`)
        extras["host_resident_stream"] = bench_stream(dev, args.stream_buckets, args.stream_bucket_mib << 20,
                                                      not args.stream_no_download)
        # the practical ceilings of 1:1, 2:1, 4:1, 1:2 and 1:4 read:write streams on this very box, measured in this very run
        cal = bench_copy(dev, args.steps, args.warmup)
        extras["copy_kernel_calibration"] = cal
        line["roofline"]["same_run_compute_free_streams"] = {
            "note": "fraction of the 8 TB/s peak that kernels with no arithmetic reach on this box in this run: plain copy, and the "
                    "block-FP8 quantiser's (2:1) and the INT4 packer's (4:1) read:write mix over contiguous 16-32 KiB pieces, and "
                    "the FP8 (1:2) and INT4 (1:4) dequantisers' mixes",
            "copy_1_to_1": cal["hbm_frac"], "fold_2_to_1": cal["compute_free_2_to_1"]["hbm_frac"],
            "fold_4_to_1": cal["compute_free_4_to_1"]["hbm_frac"], "expand_1_to_2": cal["compute_free_1_to_2"]["hbm_frac"],
            "expand_1_to_4": cal["compute_free_1_to_4"]["hbm_frac"]}
        line["other_workloads"] = extras
    # The CPU baseline runs last: its thread pool keeps spinning for a while after each parallel region, which slows
    # the launch-bound legs above (the per-parameter loop) when they run after it.
    if not args.no_cpu:
        line["cpu_baseline"], line["cpu_baseline_legs"] = cpu_baselines(
            args.cpu_seconds, (2 * r["fp8"]["elements"], 2 * r["int4"]["elements"]))
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
