#!/usr/bin/env python3
"""Benchmark of the ragged-batch decode path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one pass of the hot path over one batch of synthetic input that is
already resident in HBM.  Prints ONE JSON line.  `value` is algorithmic bytes
of a step / wall time of a step (GB/s); `roofline` prices the dominant kernel
alone (HIP events around back-to-back launches of only that kernel on the
launch stream); `cpu_baseline` is the CPU oracle timed on this box's host
cores on a bounded sample of the same workload.

Cold-HBM timing: the KV pools (or weights) are replicated so that consecutive
steps touch different memory and the replicas together exceed twice the
256 MiB Infinity Cache; the warm figure (one replica, cache-resident) is
reported beside it.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from logismos_amd import hip, kernels  # noqa: E402
from tests import workloads  # noqa: E402
from tests.gpu_harness import PagedAttnRunner, QgemvQ8Runner  # noqa: E402

HBM_PEAK_GBPS = 8000.0
COLD_BYTES = 640 << 20  # replicas together exceed 2x the 256 MiB Infinity Cache


def physical_cores() -> int:
    """Distinct (physical id, core id) pairs, the reference's way of sizing its CPU pool
    (crates/embed/src/stella.rs:474-500), capped by this process's CPU share."""
    pairs, phys, core = set(), None, None
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("physical id"):
                phys = line.split(":")[1].strip()
            elif line.startswith("core id"):
                core = line.split(":")[1].strip()
            elif not line.strip():
                if phys is not None and core is not None:
                    pairs.add((phys, core))
                phys = core = None
    except OSError:
        pass
    n = len(pairs) or (os.cpu_count() or 1)
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit():
        n = min(n, int(env))
    try:
        n = min(n, len(os.sched_getaffinity(0)))
    except AttributeError:
        pass
    return max(1, n)


def time_launches(stream, fns, steps, warmup, use_graph=True):
    """Average milliseconds per call of fns[i % len(fns)] over `steps` calls, HIP events on
    `stream`.  The timed calls are captured into one HIP graph when possible so that the host
    enqueue rate does not bound short kernels."""
    for i in range(warmup):
        fns[i % len(fns)]()
    stream.synchronize()
    e0, e1 = hip.Event(), hip.Event()
    graph = None
    if use_graph:
        try:
            g = hip.Graph(stream)
            with g:
                for i in range(steps):
                    fns[(warmup + i) % len(fns)]()
            graph = g
            graph.launch()  # one untimed replay (first launch uploads the graph)
            stream.synchronize()
        except hip.HipError:
            graph = None
    hip.synchronize()
    t0 = time.perf_counter()
    e0.record(stream)
    if graph is not None:
        graph.launch()
    else:
        for i in range(steps):
            fns[(warmup + i) % len(fns)]()
    e1.record(stream)
    e1.synchronize()
    hip.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return e0.elapsed_ms(e1) / steps, wall_ms / steps, graph is not None


def replicate(buf: hip.DeviceBuffer, copies: int):
    out = [buf]
    for _ in range(copies - 1):
        b = hip.DeviceBuffer(buf.nbytes)
        b.copy_from_device(buf, buf.nbytes)
        out.append(b)
    return out


def bench_paged_decode(args):
    import oracle as O
    case = workloads.config2()
    stream = hip.Stream()
    r = PagedAttnRunner(case, stream=stream)
    algo = workloads.paged_attn_algorithmic_bytes(case)
    kv_bytes = case["k_pool"].nbytes + case["v_pool"].nbytes
    copies = max(2, -(-COLD_BYTES // kv_bytes))
    kps, vps = replicate(r.k_pool, copies), replicate(r.v_pool, copies)

    # correctness of what is being timed (one replica, vs the oracle)
    r.launch()
    got = r.result().astype(np.float32)
    want = O.paged_attn_varlen_fp16(case["q"], case["k_pool"], case["v_pool"], case["block_tables"],
                                    case["cu_seqlens"], case["context_lens"], case["hq"],
                                    case["hkv"], case["d"], case["block_size"], case["scale"],
                                    True).astype(np.float32)
    max_abs = float(np.abs(got - want).max())

    full = [lambda k=k, v=v: r.launch(k_pool=k, v_pool=v) for k, v in zip(kps, vps)]
    dec = [lambda k=k, v=v: r.launch(phases=kernels.ATTN_PHASE_DECODE, k_pool=k, v_pool=v)
           for k, v in zip(kps, vps)]
    ms_step, wall_ms, graphed = time_launches(stream, full, args.steps, args.warmup)
    ms_dec, _, _ = time_launches(stream, dec, args.steps, args.warmup)
    ms_warm, _, _ = time_launches(stream, dec[:1], args.steps, args.warmup)

    # CPU baseline: the oracle on the same case, repeated for a bounded time
    cores = physical_cores()
    O.set_num_threads(cores)
    reps, t0 = 0, time.perf_counter()
    while True:
        O.paged_attn_varlen_fp16(case["q"], case["k_pool"], case["v_pool"], case["block_tables"],
                                 case["cu_seqlens"], case["context_lens"], case["hq"], case["hkv"],
                                 case["d"], case["block_size"], case["scale"], True)
        reps += 1
        el = time.perf_counter() - t0
        if el > args.cpu_seconds or reps >= 2000:
            break
    cpu_gbps = algo * reps / el / 1e9

    value = algo / (ms_step * 1e-3) / 1e9
    achieved = algo / (ms_dec * 1e-3) / 1e9
    return {
        "metric": "paged-attn decode achieved HBM GB/s", "value": round(value, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "config 2: ragged paged-attention decode, 16 seqs, ctx U[64,2048], "
                               "12 q / 2 kv heads, head_dim 128, block 16, fp16 KV",
                   "sum_ctx": int(case["context_lens"].sum()), "num_splits": r.num_splits,
                   "algorithmic_bytes_per_step": algo, "kv_replicas": copies,
                   "hip_graph": graphed},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "paged_attn_kernel<6,decode>", "ms_per_launch": round(ms_dec, 5),
                     "warm_cache_GBps": round(algo / (ms_warm * 1e-3) / 1e9, 1)},
        "cpu_baseline": {"value": round(cpu_gbps, 2), "unit": "GB/s", "cores": cores,
                         "kind": "port",
                         "sample": f"{reps} passes of the same config-2 batch in {el:.1f} s"},
        "parity_max_abs_vs_oracle": max_abs,
        "host_wall_ms_per_step": round(wall_ms, 5),
    }


def bench_qgemv_q8(args):
    import oracle as O
    c = workloads.config1()
    n, k = c["n"], c["k"]
    qs, d = O.quantize_q8g32(c["w"], n, k)
    stream = hip.Stream()
    r = QgemvQ8Runner(c["x"], qs, d, n, k, stream=stream)
    algo = workloads.qgemv_q8_algorithmic_bytes(n, k)
    copies = max(2, -(-COLD_BYTES // (n * k)))
    qss, ds = replicate(r.qs, copies), replicate(r.d, copies)
    r.launch()
    want = O.qgemv_q8g32_f32(c["x"], qs, d, n, k)
    max_abs = float(np.abs(r.result() - want).max())

    def mk(q, dd):
        return lambda: kernels.launch_qgemv_q8g32_f32(r.x, q, dd, r.y, n, k, stream)
    cold = [mk(q, dd) for q, dd in zip(qss, ds)]
    ms_cold, _, graphed = time_launches(stream, cold, args.steps, args.warmup)
    ms_warm, _, _ = time_launches(stream, cold[:1], args.steps, args.warmup)
    cores = physical_cores()
    O.set_num_threads(cores)
    reps, t0 = 0, time.perf_counter()
    while True:
        O.qgemv_q8g32_f32(c["x"], qs, d, n, k)
        reps += 1
        el = time.perf_counter() - t0
        if el > args.cpu_seconds / 2 or reps >= 20000:
            break
    return {"workload": "config 1: Q8G32 GEMV 8960x1536, x f32", "algorithmic_bytes": algo,
            "ms_per_launch_cold": round(ms_cold, 5), "GBps_cold": round(algo / ms_cold / 1e6, 1),
            "frac_of_peak_cold": round(algo / ms_cold / 1e6 / HBM_PEAK_GBPS, 4),
            "GBps_warm_cache": round(algo / ms_warm / 1e6, 1), "weight_replicas": copies,
            "hip_graph": graphed, "parity_max_abs_vs_oracle": max_abs,
            "cpu_baseline_GBps": round(algo * reps / el / 1e9, 2), "cpu_cores": cores}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; every workload is the full single-GPU "
                 "shape and nothing here uses a second device (--gpus must be 1)")
    if hip.device_count() < 1:
        sys.exit("bench.py: no HIP device visible; there is no CPU fallback to time")
    hip.set_device(0)
    kernels.library()
    line = bench_paged_decode(args)
    line["qgemv_q8"] = bench_qgemv_q8(args)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
