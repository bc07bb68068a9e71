#!/usr/bin/env python3
"""Benchmark of the ragged-batch decode path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one continuous-batching decode step (config 5 of the baseline: 32
live sequences, Qwen3-8B-style geometry) over synthetic inputs already resident
in HBM.  Prints ONE JSON line.  `value` is decode tokens per second;
`roofline` prices the dominant kernel alone (HIP events around back-to-back
launches of only the paged-attention decode kernel on the launch stream);
`cpu_baseline` is the CPU oracle timed on this box's host cores on a bounded
sample of the same workload.  The per-kernel legs (configs 1-4) are reported in
the same line under their own keys.

Cold-HBM timing: the KV pools (or weights) are replicated so that consecutive
steps touch different memory and the replicas together exceed twice the
256 MiB Infinity Cache; the warm figure (one replica, cache-resident) is
reported beside it.
"""
from __future__ import annotations

import argparse
import ctypes as C
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
PMC_CAL_BYTES = 256 << 20  # bytes the calibration copy reads (and writes)
PARITY_REL_L2_BOUND = 4e-3  # one layer of the step vs the oracle (bf16 intermediates)
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


def measured_traffic(summary: str, key: str = "traffic_bytes_per_launch:"):
    """HBM bytes per launch from a committed hardware-counter summary under profiles/ (the
    counters cannot be read from inside this process); None when there is none."""
    try:
        with open(os.path.join(ROOT, "profiles", summary)) as f:
            for ln in f:
                if ln.strip().startswith(key):
                    return int(ln.split(":")[1])
    except OSError:
        pass
    return None


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


_CEILING_CACHE: dict[int, dict] = {}


def read_ceiling(stream, nbytes: int) -> dict:
    """What a read-only kernel reaches on THIS box for a launch of `nbytes` (GB/s): the best
    of plain / non-temporal 16-byte loads in two work splits, over distinct replicas that
    together exceed twice the Infinity Cache, timed like the legs themselves (HIP events around a captured graph of
    back-to-back launches).  The datasheet's 8 TB/s is the peak every fraction is quoted
    against; this is the ceiling a launch of that size can actually be held to."""
    nbytes = max(1 << 16, int(nbytes) // 4096 * 4096)
    if nbytes not in _CEILING_CACHE:
        copies = max(2, min(64, -(-COLD_BYTES // nbytes)))
        buf = hip.DeviceBuffer(nbytes * copies)
        buf.fill(0x5A)
        sink = hip.DeviceBuffer(16)
        launches = 200 if nbytes < (64 << 20) else 40
        rates = {}
        for name, flags in (("plain", 0), ("non_temporal", kernels.PROBE_NON_TEMPORAL),
                            ("plain_strided", kernels.PROBE_STRIDED),
                            ("non_temporal_strided",
                             kernels.PROBE_NON_TEMPORAL | kernels.PROBE_STRIDED)):
            fns = [lambda i=i, flags=flags: kernels.launch_probe_read(
                buf.offset(i * nbytes), sink, nbytes, stream, flags) for i in range(copies)]
            ms, _, _ = time_launches(stream, fns, launches, 8)
            rates[name] = round(nbytes / ms / 1e6, 1)
        del buf
        _CEILING_CACHE[nbytes] = {"GBps": max(rates.values()), "bytes": nbytes, **rates}
    return _CEILING_CACHE[nbytes]


def against_ceiling(stream, nbytes: int, achieved_gbps: float) -> dict:
    """The two fields every HBM-bound figure carries beside its fraction of the 8 TB/s peak."""
    c = read_ceiling(stream, nbytes)
    return {"measured_read_ceiling_GBps": c["GBps"],
            "frac_of_measured_ceiling": round(achieved_gbps / c["GBps"], 4)}


_MFMA_CEILING_CACHE = {}


def mfma_ceiling(stream, bf16: bool) -> dict:
    """What the matrix cores of THIS box sustain (TFLOP/s) when a kernel issues nothing but
    v_mfma_f32_32x32x16 on every CU: with operands that never change, and with operands
    rewritten between the MFMAs as real data rewrites them.  The datasheet's 2.5 PFLOP/s is
    the peak every fraction is quoted against; the second figure is the ceiling an MFMA-bound
    kernel on real data can actually be held to (the part slows the pipes when their inputs
    toggle)."""
    if bf16 not in _MFMA_CEILING_CACHE:
        sink = hip.DeviceBuffer(16)
        iters = 4000
        flops = kernels.probe_mfma_flops(iters)
        rates = {}
        for name, flags in (("constant_operands", 0), ("changing_operands",
                                                       kernels.PROBE_MFMA_CHANGING)):
            flags |= kernels.PROBE_MFMA_BF16 if bf16 else 0
            fn = [lambda flags=flags: kernels.launch_probe_mfma(sink, iters, flags, stream)]
            ms, _, _ = time_launches(stream, fn, 10, 3)
            rates[name] = round(flops / ms / 1e9, 1)
            rates[name + "_board_W"], rates["board_power_cap_W"] = board_power_watts(stream, fn[0])
        _MFMA_CEILING_CACHE[bf16] = rates
    return _MFMA_CEILING_CACHE[bf16]


def board_power_watts(stream, launch, seconds: float = 1.5):
    """Board power (W, mean of the second half of the samples) while `launch` loops for
    `seconds`, and the board's power cap, both read from the amdgpu hwmon node; (None, None)
    where the node is not readable.  The probe's and the GEMM's figures beside the cap say
    whether a kernel runs into the cap -- below it the clock holds 2.4 GHz, at it the part
    lowers the clock."""
    import glob
    import threading
    nodes = glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input") or \
        glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average")
    if not nodes:
        return None, None

    def read(path):
        try:
            with open(path) as f:
                return int(f.read()) / 1e6
        except (OSError, ValueError):
            return None
    cap = read(os.path.join(os.path.dirname(nodes[0]), "power1_cap"))
    samples, stop = [], threading.Event()

    def poll():
        while not stop.is_set():
            w = read(nodes[0])
            if w is not None:
                samples.append(w)
            time.sleep(0.05)
    t = threading.Thread(target=poll)
    t.start()
    t0 = time.time()
    while time.time() - t0 < seconds:
        for _ in range(5):
            launch()
        stream.synchronize()
    stop.set()
    t.join()
    tail = samples[len(samples) // 2:]
    return (round(sum(tail) / len(tail), 0) if tail else None), cap


def against_mfma_ceiling(stream, bf16: bool, achieved_tflops: float) -> dict:
    """The fields every MFMA-bound figure carries beside its fraction of the 2.5 PFLOP/s peak."""
    c = mfma_ceiling(stream, bf16)
    return {"measured_mfma_ceiling_TFLOPs": c["changing_operands"],
            "measured_mfma_rate_constant_operands_TFLOPs": c["constant_operands"],
            "frac_of_measured_ceiling": round(achieved_tflops / c["changing_operands"], 4),
            "board_power_W": {"cap": c["board_power_cap_W"],
                              "mfma_probe_constant_operands": c["constant_operands_board_W"],
                              "mfma_probe_changing_operands": c["changing_operands_board_W"]}}


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
                     "kernel": "paged_attn_kernel<6> (static split; a batch this small stays off the "
                               "balanced kernel)", "ms_per_launch": round(ms_dec, 5),
                     "warm_cache_GBps": round(algo / (ms_warm * 1e-3) / 1e9, 1),
                     **against_ceiling(stream, algo, achieved),
                     "target_70pct_of_peak": "met" if achieved >= 0.7 * HBM_PEAK_GBPS
                     else "missed"},
        "cpu_baseline": {"value": round(cpu_gbps, 2), "unit": "GB/s", "cores": cores,
                         "kind": "port",
                         "sample": f"{reps} passes of the same config-2 batch in {el:.1f} s"},
        "parity_max_abs_vs_oracle": max_abs,
        "host_wall_ms_per_step": round(wall_ms, 5),
    }


def bench_mixed_config4(args):
    """Config 4: 48 decode rows + 16 prefill chunks of 512 tokens in one packed token buffer.
    One step = GPU-side packing (cu_seqlens, slot mapping, context lengths), the K/V rows of
    the new tokens scattered into the paged pools, ragged attention over the whole batch."""
    import oracle as O
    case = workloads.config4()
    stream = hip.Stream()
    rng = np.random.default_rng(99)
    S = len(case["new_tokens"])
    T = int(case["cu_seqlens"][-1])
    row = case["hkv"] * case["d"]
    k_new = rng.standard_normal((T, row), np.float32).astype(np.float16)
    v_new = rng.standard_normal((T, row), np.float32).astype(np.float16)
    cu_h, slots_h, ctx_h, _ = O.pack_ragged(case["new_tokens"], case["prior_ctx"],
                                            case["block_tables"], case["block_size"])
    # the attention runner reads what the packer wrote on the GPU, not host-built copies
    r = PagedAttnRunner(case, stream=stream)
    d_new = hip.DeviceBuffer.from_numpy(case["new_tokens"])
    d_prior = hip.DeviceBuffer.from_numpy(case["prior_ctx"])
    d_slots = hip.DeviceBuffer(T * 8)
    r.cu.fill(0xFF)
    r.ctx.fill(0xFF)
    d_knew = hip.DeviceBuffer.from_numpy(k_new)
    d_vnew = hip.DeviceBuffer.from_numpy(v_new)

    def pack():
        kernels.launch_pack_ragged(d_new, d_prior, r.bt, r.cu, d_slots, r.ctx, S,
                                   case["block_size"], case["max_blocks"], stream)

    def write():
        kernels.launch_kv_write_fp16(d_knew, d_vnew, r.k_pool, r.v_pool, d_slots, T, case["hkv"],
                                     case["d"], stream)

    def step():
        pack()
        write()
        r.launch()

    step()
    got = r.result()
    pack_ok = (np.array_equal(r.cu.to_numpy(np.int32, (S + 1,)), cu_h)
               and np.array_equal(d_slots.to_numpy(np.int64, (T,)), slots_h)
               and np.array_equal(r.ctx.to_numpy(np.int32, (S,)), ctx_h))
    # parity sample: the prefill chunk with the shortest context and three decode rows, as a
    # reduced batch for the oracle over the pools with the new rows written
    kp, vp = case["k_pool"].copy(), case["v_pool"].copy()
    kp[slots_h] = k_new
    vp[slots_h] = v_new
    pre = [s for s in range(S) if case["new_tokens"][s] > 1]
    dec = [s for s in range(S) if case["new_tokens"][s] == 1]
    pick = [min(pre, key=lambda s: case["context_lens"][s])] + \
        sorted(dec, key=lambda s: case["context_lens"][s])[:3]
    sub_q = np.concatenate([case["q"][cu_h[s]:cu_h[s + 1]] for s in pick])
    sub_cu = np.concatenate([[0], np.cumsum(case["new_tokens"][pick])]).astype(np.int32)
    want = O.paged_attn_varlen_fp16(sub_q, kp, vp, case["block_tables"][pick], sub_cu,
                                    case["context_lens"][pick], case["hq"], case["hkv"],
                                    case["d"], case["block_size"], case["scale"], True)
    sub_got = np.concatenate([got[cu_h[s]:cu_h[s + 1]] for s in pick])
    max_abs = float(np.abs(sub_got.astype(np.float32) - want.astype(np.float32)).max())

    steps, warmup = max(10, args.steps // 10), 3
    ms_step, wall_ms, graphed = time_launches(stream, [step], steps, warmup)
    ms_pack, _, _ = time_launches(stream, [pack], steps, warmup)
    ms_write, _, _ = time_launches(stream, [write], steps, warmup)
    ms_pre, _, _ = time_launches(
        stream, [lambda: r.launch(phases=kernels.ATTN_PHASE_PREFILL)], steps, warmup)
    ms_dec, _, _ = time_launches(
        stream, [lambda: r.launch(phases=kernels.ATTN_PHASE_DECODE)], steps, warmup)
    ms_merge, _, _ = time_launches(
        stream, [lambda: r.launch(phases=kernels.ATTN_PHASE_MERGE)], steps, warmup)

    # board power while the prefill kernel loops: says whether it runs into the power cap, as
    # the tiled GEMM does, or waits for something else at full clock
    pre_watts, _ = board_power_watts(
        stream, lambda: r.launch(phases=kernels.ATTN_PHASE_PREFILL), 1.5)

    is_dec = case["new_tokens"] == 1
    sub = lambda m: {**case, "new_tokens": case["new_tokens"][m],  # noqa: E731
                     "context_lens": case["context_lens"][m]}
    flops_pre = workloads.paged_attn_flops(sub(~is_dec))
    # HBM bytes of the prefill kernel: the committed counter summary, if it was taken at this
    # workload's byte count (every K/V row of the chunk sequences once, q in, out out)
    pre_ctx = case["context_lens"][~is_dec].astype(np.int64)
    pre_new = case["new_tokens"][~is_dec].astype(np.int64)
    pre_bytes = int(pre_ctx.sum()) * 2 * row * 2 + 2 * int(pre_new.sum()) * case["hq"] * 128 * 2
    prefill_traffic = measured_traffic("paged_attn_prefill_config4_pmc.txt")
    if measured_traffic("paged_attn_prefill_config4_pmc.txt",
                        "algorithmic_bytes_per_launch:") != pre_bytes:
        prefill_traffic = None
    ctx_dec = case["context_lens"][is_dec].astype(np.int64)
    dec_bytes = int(ctx_dec.sum()) * 2 * row * 2
    return {
        "metric": "mixed chunked-prefill + decode attention step, new tokens/s",
        "value": round(T / (ms_step * 1e-3), 1), "unit": "tokens/s",
        "ms_per_step": round(ms_step, 4), "steps": steps, "warmup": warmup, "dtype": "f16",
        "config": {"workload": "config 4: 48 decode rows (ctx log-uniform 128..32768) + 16 prefill "
                               "chunks x 512 tokens (prior 0..8192), 32 q / 8 kv heads, head_dim "
                               "128, block 16; one layer's packing + KV write + attention",
                   "total_new_tokens": T, "sum_ctx": int(case["context_lens"].sum()),
                   "num_splits": r.num_splits, "hip_graph": graphed},
        "kernels_ms": {"pack_ragged": round(ms_pack, 4), "kv_write": round(ms_write, 4),
                       "prefill": round(ms_pre, 4), "decode": round(ms_dec, 4),
                       "merge": round(ms_merge, 4)},
        "roofline": {"bound": "mfma", "achieved": round(flops_pre / (ms_pre * 1e-3) / 1e12, 1),
                     "peak": 2500.0, "unit": "TFLOP/s",
                     "frac": round(flops_pre / (ms_pre * 1e-3) / 1e12 / 2500.0, 4),
                     "traffic": prefill_traffic, "kernel": "paged_attn_prefill_kernel<4>",
                     "flops_per_launch": flops_pre,
                     **against_mfma_ceiling(stream, False,
                                            flops_pre / (ms_pre * 1e-3) / 1e12),
                     "board_power_W_during": pre_watts},
        "decode_rows_GBps": round(dec_bytes / (ms_dec * 1e-3) / 1e9, 1),
        "decode_rows_frac_of_peak": round(dec_bytes / (ms_dec * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        "decode_rows": against_ceiling(stream, dec_bytes, dec_bytes / (ms_dec * 1e-3) / 1e9),
        "gpu_packing_bit_exact": bool(pack_ok),
        "parity_max_abs_vs_oracle": max_abs,
        "parity_sample": f"sequences {pick} (1 prefill chunk, 3 decode rows)",
    }


def bench_turbo3(args):
    """One layer's decode attention of config 5 over TurboQuant 3-bit pools (56 bytes per
    head row instead of 256), next to the fp16 pools it was encoded from."""
    case = workloads.config5_attention()
    stream = hip.Stream()
    S, hq, hkv = len(case["context_lens"]), case["hq"], case["hkv"]
    r = PagedAttnRunner(case, stream=stream)
    rows = case["k_pool"].shape[0]
    slots = hip.DeviceBuffer.from_numpy(np.arange(rows, dtype=np.int64))
    copies = 3   # 3 x 2 x 0.3 GB of fp16 pools > 2 x Infinity Cache
    kps, vps = replicate(r.k_pool, copies), replicate(r.v_pool, copies)
    t3 = []
    for k, v in zip(kps, vps):
        kp, vp = hip.DeviceBuffer(rows * hkv * 56), hip.DeviceBuffer(rows * hkv * 56)
        kernels.launch_kv_write_turbo3(k, v, kp, vp, slots, rows, hkv, stream)
        t3.append((kp, vp))
    stream.synchronize()
    ns = r.num_splits

    def turbo(kp, vp):
        return lambda: kernels.launch_paged_attn_varlen_turbo3(
            r.q, kp, vp, r.bt, r.cu, r.ctx, r.out, r.ws, S, S, 1, hq, hkv, case["block_size"],
            case["max_blocks"], ns, case["scale"], stream)
    ms16, _, _ = time_launches(stream, [(lambda k=k, v=v: r.launch(k_pool=k, v_pool=v))
                                        for k, v in zip(kps, vps)], 60, 6)
    ms3, _, _ = time_launches(stream, [turbo(k, v) for k, v in t3], 60, 6)
    ctx = int(case["context_lens"].sum())
    return {"workload": "config 5 attention (32 seqs, ctx U[256,8192], 32 q / 8 kv heads), one "
                        "layer, decode + merge; turbo3 = TurboQuant 3-bit KV, decode fused",
            "sum_ctx": ctx,
            "fp16": {"us": round(ms16 * 1e3, 1), "kv_bytes": ctx * 4096,
                     "GBps": round(ctx * 4096 / ms16 / 1e6, 1),
                     **against_ceiling(stream, ctx * 4096, ctx * 4096 / ms16 / 1e6)},
            "turbo3": {"us": round(ms3 * 1e3, 1), "kv_bytes": ctx * 896,
                       "GBps": round(ctx * 896 / ms3 / 1e6, 1),
                       **against_ceiling(stream, ctx * 896, ctx * 896 / ms3 / 1e6)},
            "keys_per_us": {"fp16": round(ctx / (ms16 * 1e3), 1),
                            "turbo3": round(ctx / (ms3 * 1e3), 1)}}


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
            **against_ceiling(stream, algo, algo / ms_cold / 1e6),
            "target_70pct_of_peak": "met" if algo / ms_cold / 1e6 >= 0.7 * HBM_PEAK_GBPS
            else "missed",
            "GBps_warm_cache": round(algo / ms_warm / 1e6, 1), "weight_replicas": copies,
            "hip_graph": graphed, "parity_max_abs_vs_oracle": max_abs,
            "cpu_baseline_GBps": round(algo * reps / el / 1e9, 2), "cpu_cores": cores}


def bench_q4(args):
    """Config 3: Q4G128 12288x4096 at batch 1..16 (cold weights)."""
    import oracle as O
    rng = np.random.default_rng(workloads.SEED + 3)
    n, k = 12288, 4096
    qw = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    s = (rng.random((n, k // 128), np.float32) * 0.004 + 0.004).astype(np.float16)
    z = (rng.random((n, k // 128), np.float32) * 2 + 6.5).astype(np.float16)
    x = O.f32_to_bf16_bits(rng.standard_normal((16, k), np.float32))
    stream = hip.Stream()
    out = {}
    from tests.gpu_harness import QgemmQ4Runner
    for b in (1, 2, 4, 8, 16):
        r = QgemmQ4Runner(x[:b], qw, s, z, b, n, k, stream=stream)
        copies = max(2, -(-COLD_BYTES // qw.nbytes))
        qws = replicate(r.qw, copies)
        algo = workloads.qgemm_q4_algorithmic_bytes(b, n, k)
        ms, _, _ = time_launches(stream, [(lambda q=q: r.launch(qw=q)) for q in qws], args.steps,
                                 args.warmup)
        # the same launches on one replica: the weights (27 MB) stay in the caches
        ms_warm, _, _ = time_launches(stream, [lambda: r.launch()], args.steps, args.warmup)
        out[f"b{b}"] = {"us": round(ms * 1e3, 2), "GBps": round(algo / ms / 1e6, 1),
                        "frac_of_peak": round(algo / ms / 1e6 / HBM_PEAK_GBPS, 4),
                        **against_ceiling(stream, workloads.qgemm_q4_algorithmic_bytes(1, n, k),
                                          algo / ms / 1e6),
                        "target_70pct_of_peak": "met" if algo / ms / 1e6 >= 0.7 * HBM_PEAK_GBPS
                        else "missed",
                        "GBps_warm_cache": round(algo / ms_warm / 1e6, 1),
                        "kernel": ("gemv (VALU dot2)" if b <= 1
                                   else "mfma, x in registers, weights through an LDS ring")}
        del r, qws
    # the same matrix size as ggml Q4_0 weights through the Q4G32 GEMV (x fp32, batch 1)
    qw32 = hip.DeviceBuffer.from_numpy(qw)
    sc32 = hip.DeviceBuffer.from_numpy(
        (rng.random((n, k // 32), np.float32) * 0.004 + 0.004).astype(np.float16))
    mn32 = hip.DeviceBuffer.from_numpy(
        (rng.random((n, k // 32), np.float32) * -0.06).astype(np.float16))
    x32 = hip.DeviceBuffer.from_numpy(rng.standard_normal(k, np.float32))
    y32 = hip.DeviceBuffer(n * 4)
    qws = replicate(qw32, max(2, -(-COLD_BYTES // qw.nbytes)))
    algo32 = n * k // 2 + n * (k // 32) * 4 + 4 * k + 4 * n
    ms, _, _ = time_launches(
        stream, [(lambda q=q: kernels.launch_qgemv_q4g32_f32(x32, q, sc32, mn32, y32, n, k, stream))
                 for q in qws], args.steps, args.warmup)
    ms_warm, _, _ = time_launches(
        stream, [lambda: kernels.launch_qgemv_q4g32_f32(x32, qw32, sc32, mn32, y32, n, k, stream)],
        args.steps, args.warmup)
    out["q4g32_b1"] = {"us": round(ms * 1e3, 2), "GBps": round(algo32 / ms / 1e6, 1),
                       "GBps_warm_cache": round(algo32 / ms_warm / 1e6, 1),
                       "kernel": "qgemv_q4g32 (ggml Q4_0/Q4_1 arithmetic, x fp32)"}
    # ... and as a batch of 16 bf16 rows through the matrix-core kernel
    for b in (4, 16):
        xb = hip.DeviceBuffer.from_numpy(O.f32_to_bf16_bits(rng.standard_normal((b, k), np.float32)))
        yb = hip.DeviceBuffer(b * n * 2)
        algo = n * k // 2 + n * (k // 32) * 4 + 2 * b * k + 2 * b * n
        ms, _, _ = time_launches(
            stream, [(lambda q=q: kernels.launch_qgemm_q4g32_bf16(xb, q, sc32, mn32, yb, b, n, k,
                                                                  stream)) for q in qws],
            args.steps, args.warmup)
        out[f"q4g32_b{b}"] = {"us": round(ms * 1e3, 2), "GBps": round(algo / ms / 1e6, 1),
                              "kernel": "qgemm_q4g32 (mfma, one group per 16x16x32 product)"}
    return {"workload": "config 3: Q4G128 GEMV/GEMM 12288x4096, x bf16, cold weights", **out}


def bench_q4_tall(args):
    """Config 4's packed token buffer (48 decode rows + 16 x 512 prefill rows = 8240 rows) through
    one layer's four Q4G128 projections at Qwen3-8B geometry: `linear_t` at m = 8240 on the
    tiled matrix-core kernel.  MFMA-bound by construction (arithmetic intensity ~4000 flop per
    weight byte); reported against the dense bf16 peak."""
    import oracle as O
    stream = hip.Stream()
    rng = np.random.default_rng(workloads.SEED + 40)
    b = 8240
    shapes = [("qkv", 6144, 4096), ("o", 4096, 4096), ("gate_up", 24576, 4096),
              ("down", 4096, 12288)]
    out, flops_all, ms_all, ms_noworkspace = {}, 0.0, 0.0, 0.0
    parity, power = None, {}
    for name, n, k in shapes:
        qw = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
        s = (rng.random((n, k // 128), np.float32) * 0.004 + 0.004).astype(np.float16)
        z = (rng.random((n, k // 128), np.float32) * 2 + 6.5).astype(np.float16)
        xb = O.f32_to_bf16_bits(rng.standard_normal((b, k), np.float32))
        d = [hip.DeviceBuffer.from_numpy(a) for a in (xb, qw, s.view(np.uint16), z.view(np.uint16))]
        dy = hip.DeviceBuffer(b * n * 2)
        ws = hip.DeviceBuffer(kernels.qgemm_q4g128_tall_workspace_bytes(b, k))
        # the entry point with a workspace (first pass over x + the tiled kernel) ...
        fn = lambda: kernels.launch_qgemm_q4g128_tall(d[0], d[1], d[2], d[3], dy, ws, b, n, k,  # noqa: E731
                                                      stream)
        # ... and the same product through the entry point without one
        fn0 = lambda: kernels.launch_qgemm_q4g128_bf16(d[0], d[1], d[2], d[3], dy, b, n, k, stream)  # noqa: E731
        ms0, _, _ = time_launches(stream, [fn0], 10, 2)
        ms, _, _ = time_launches(stream, [fn], 10, 2)
        ms_noworkspace += ms0
        if name == "o":
            # parity of what is being timed: a sample of rows against the oracle
            rows = np.r_[0:4, 4111:4115, 8236:8240]
            got = O.bf16_bits_to_f32(dy.to_numpy(np.uint16, (b, n))[rows])
            want = O.bf16_bits_to_f32(O.qgemm_q4g128_bf16(xb[rows], qw, s, z, len(rows), n, k))
            parity = float(np.abs(got - want).max())
        flops = 2.0 * b * n * k
        flops_all += flops
        ms_all += ms
        out[name] = {"n": n, "k": k, "us": round(ms * 1e3, 1),
                     "TFLOPs": round(flops / ms / 1e9, 1)}
        if name == "gate_up":
            # the same launch on x = 0: operands of the A side that never toggle, the kernel's
            # schedule without what the board's power cap takes off the clock
            power["gate_up"], _ = board_power_watts(stream, fn)
            d0 = hip.DeviceBuffer.from_numpy(np.zeros_like(xb))
            fz = lambda: kernels.launch_qgemm_q4g128_tall(d0, d[1], d[2], d[3], dy, ws, b, n, k,  # noqa: E731
                                                          stream)
            msz, _, _ = time_launches(stream, [fz], 10, 2)
            power["gate_up_x_zero"], _ = board_power_watts(stream, fz)
            out[name]["us_x_zero"] = round(msz * 1e3, 1)
            del d0
        del d, dy, ws
    return {"workload": "config 4's 8240 packed rows through one layer's Q4G128 projections "
                        "(qkv 6144x4096, o 4096x4096, gate_up 24576x4096, down 4096x12288)",
            "kernel": "q4_tall_prepare_kernel + qgemm_q4g128_tallp_kernel (128x256 tiles, x and "
                      "weights straight into a three-deep LDS ring, v_mfma_f32_32x32x16_bf16; the "
                      "tiles of the last partial round of workgroups split over K + "
                      "q4_tall_reduce_kernel)",
            "projections": out, "ms_per_layer": round(ms_all, 4),
            "ms_per_layer_entry_point_without_workspace": round(ms_noworkspace, 4),
            "roofline": {"bound": "mfma", "achieved": round(flops_all / ms_all / 1e9, 1),
                         "peak": 2500.0, "unit": "TFLOP/s",
                         "frac": round(flops_all / ms_all / 1e9 / 2500.0, 4), "traffic": None,
                         "flops_per_layer": flops_all,
                         **against_mfma_ceiling(stream, True, flops_all / ms_all / 1e9)},
            "board_power_W_during": power,
            "parity_max_abs_vs_oracle_sample": parity}


def bench_mixed_step_config4(args):
    """Config 4's packed batch (48 decode rows + 16 prefill chunks of 512 tokens = 8240 rows)
    through the whole step executor at Qwen3-8B geometry, 36 layers: the rows go through the
    tiled Q4G128 GEMMs, rope + KV write, the chunked-prefill and decode attention kernels and
    the small operators over all rows.  Timing only: the executor's many-row path is held
    against the oracle at a few hundred rows in tests/ (a layer of 8240 rows on the CPU oracle
    takes minutes); random nibbles as weights, pools of repeated random rows."""
    from tests.gpu_harness import DecodeStepRunner
    rng = np.random.default_rng(workloads.SEED + 44)
    L, hidden, hq, hkv, inter = 36, 4096, 32, 8, 12288
    c4 = workloads.config4()
    new = c4["new_tokens"].astype(np.int32)
    ctx = c4["context_lens"].astype(np.int32)
    del c4
    cfg, layers, batch = workloads.decode_step_problem(
        rng, 1, hidden, hq, hkv, inter, ctx, new_tokens=new, random_nibbles=True,
        pool_period_rows=8191)
    stream = hip.Stream()
    r = DecodeStepRunner(cfg, layers * L, batch, stream=stream, share_layer_data=True)
    del layers
    for _ in range(2):
        r.launch()
    stream.synchronize()
    steps = 3
    e0, e1 = hip.Event(), hip.Event()
    e0.record(stream)
    for _ in range(steps):
        r.launch()
    e1.record(stream)
    e1.synchronize()
    ms = e0.elapsed_ms(e1) / steps
    out = O_bf16_finite(r)
    rows = int(new.sum())
    return {"workload": "config 4's mixed batch through the step executor: 64 sequences, "
                        f"{rows} packed rows (48 decode + 16 x 512 prefill), sum of contexts "
                        f"{int(ctx.sum())}, {L} layers at hidden {hidden}, {hq}/{hkv} heads, MLP "
                        f"{inter}, Q4G128 weights, fp16 paged KV",
            "ms_per_step": round(ms, 2), "ms_per_layer": round(ms / L, 3),
            "new_tokens_per_s": round(rows / ms * 1e3, 0), "outputs_finite": out,
            "parity": "not checked at this size (minutes on the CPU oracle); the same code path "
                      "is checked against the oracle at 142-200 rows in "
                      "tests/test_gpu_decode_step.py and per operator in "
                      "tests/test_gpu_decode_step_many_rows_operators.py"}


def O_bf16_finite(r) -> bool:
    import oracle as O
    return bool(np.isfinite(O.bf16_bits_to_f32(r.result_bits())).all())


def bench_decode_step(args):
    """Config 5: full decode step, Qwen3-8B-style geometry, 32 live sequences."""
    import oracle as O
    from oracle import decode_step as OS
    from tests.gpu_harness import DecodeStepRunner
    rng = np.random.default_rng(workloads.SEED + 5)
    S, L, hidden, hq, hkv, inter, bs = 32, 36, 4096, 32, 8, 12288, 16
    steps, warmup = args.steps_c5, args.warmup_c5
    total_steps = steps + warmup + 2
    ctx0 = rng.integers(256, 8193, size=S).astype(np.int64)
    # per-step contexts: every sequence grows by one token per step; each step one sequence
    # finishes and a new one (context U[256,8192], its prefill not part of the step) takes
    # its row and its blocks
    ctx_steps = np.zeros((total_steps, S), np.int64)
    cur = ctx0.copy()
    for i in range(total_steps):
        cur[i % S] = rng.integers(256, 8193)
        ctx_steps[i] = cur
        cur = cur + 1
    max_ctx = int(ctx_steps.max()) + 1
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=1, hidden=hidden, hq=hq, hkv=hkv, inter=inter,
        ctx=np.full(S, max_ctx), max_pos=max_ctx + 1, random_nibbles=True)
    max_blocks = batch["block_tables"].shape[1]
    stream = hip.Stream()

    # ---- CPU baseline + parity on a bounded sample: ONE layer of step 0
    b0 = dict(batch, h=batch["h"].copy())
    prior0 = (ctx_steps[0] - 1).astype(np.int32)
    cu, slots, ctx_l, _ = O.pack_ragged(np.ones(S, np.int32), prior0, batch["block_tables"], bs)
    b0.update(cu_seqlens=cu, slots=slots, context_lens=ctx_l, positions=prior0)
    g1 = DecodeStepRunner(cfg, layers, b0, stream=stream)
    g1.launch()
    got = O.bf16_bits_to_f32(g1.result_bits())
    del g1
    cores = physical_cores()
    O.set_num_threads(cores)
    import copy
    lay_cpu = copy.deepcopy(layers)
    want = O.bf16_bits_to_f32(OS.decode_step(cfg, lay_cpu, dict(b0, h=batch["h"].copy())))
    rel_l2 = float(np.linalg.norm(got - want) / np.linalg.norm(want))
    if not (rel_l2 < PARITY_REL_L2_BOUND):
        sys.exit(f"bench.py: the one-layer step differs from the CPU oracle by relative L2 "
                 f"{rel_l2:.3e} (bound {PARITY_REL_L2_BOUND:.0e}); a throughput of wrong results "
                 "is not reported")
    # the baseline: one whole step (36 layers) on the oracle; the 36 layers share one layer's
    # weights and pools (36 sets of pools would be 38 GB of host memory), which leaves the
    # arithmetic and the bytes touched per layer as they are
    t0 = time.perf_counter()
    OS.decode_step(cfg, lay_cpu * L, dict(b0, h=batch["h"].copy()))
    cpu_s = time.perf_counter() - t0
    del lay_cpu

    # ---- the 36-layer problem on the device (layer data replicated device-to-device)
    r = DecodeStepRunner(cfg, layers * L, b0, stream=stream, share_layer_data=True)
    d_prior = hip.DeviceBuffer.from_numpy((ctx_steps - 1).astype(np.int32))   # [steps][S]
    d_ones = hip.DeviceBuffer.from_numpy(np.ones(S, np.int32))
    d_cur_prior = r.idx["positions"]    # positions == prior context of the new token

    def one_step(i, graph):
        d_cur_prior.copy_from_device_async(d_prior, 4 * S, stream, src_offset=4 * S * i)
        graph.launch()

    g = hip.Graph(stream)
    with g:
        kernels.launch_pack_ragged(d_ones, d_cur_prior, r.idx["block_tables"],
                                   r.idx["cu_seqlens"], r.slots, r.idx["context_lens"], S, bs,
                                   max_blocks, stream)
        r.launch()
    for i in range(warmup):
        one_step(i, g)
    stream.synchronize()
    e0, e1 = hip.Event(), hip.Event()
    hip.synchronize()
    t0 = time.perf_counter()
    e0.record(stream)
    for i in range(steps):
        one_step(warmup + i, g)
    e1.record(stream)
    e1.synchronize()
    hip.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ms_step = e0.elapsed_ms(e1) / steps

    # ---- the dominant kernel alone: paged-attention decode at this shape, rotating layers
    sum_ctx = float(ctx_steps[warmup:warmup + steps].sum()) / steps
    c_attn = dict(q=np.zeros((S, hq, 128), np.float16), hq=hq, hkv=hkv, d=128, block_size=bs,
                  max_blocks=max_blocks, scale=1.0 / np.sqrt(128.0))
    d_q = hip.DeviceBuffer(S * hq * 128 * 2)
    d_q.fill(0x3C)
    d_o = hip.DeviceBuffer(S * hq * 128 * 2)
    ns = r.num_splits
    d_ws = hip.DeviceBuffer(max(16, kernels.paged_attn_workspace_bytes(S, hq, 128, ns)))

    def attn(l):
        kp, vp = r.pools[l]
        return lambda: kernels.launch_paged_attn_varlen_fp16(
            d_q, kp, vp, r.idx["block_tables"], r.idx["cu_seqlens"], r.idx["context_lens"], d_o,
            d_ws, S, S, 1, hq, hkv, 128, bs, max_blocks, ns, c_attn["scale"], True, stream,
            kernels.ATTN_PHASE_DECODE)
    # ... at the contexts of step 0, so that the bytes per launch do not depend on how many
    # steps were timed before
    d_cur_prior.copy_from_device_async(d_prior, 4 * S, stream)
    kernels.launch_pack_ragged(d_ones, d_cur_prior, r.idx["block_tables"], r.idx["cu_seqlens"],
                               r.slots, r.idx["context_lens"], S, bs, max_blocks, stream)
    stream.synchronize()
    ctx_now = r.idx["context_lens"].to_numpy(np.int32, (S,)).astype(np.int64)
    assert np.array_equal(ctx_now, ctx_steps[0])
    attn_bytes = int(ctx_now.sum()) * 2 * hkv * 128 * 2 + 2 * S * hq * 128 * 2 + \
        4 * int(((ctx_now + bs - 1) // bs).sum()) + 4 * (2 * S + 1)
    ms_attn, _, _ = time_launches(stream, [attn(l) for l in range(L)], 72, 8)
    # one plain copy of known size (outside every timed region): the dispatch that hardware
    # counter runs of this command are scaled by
    cal = hip.DeviceBuffer(2 * PMC_CAL_BYTES)
    cal.fill(0x11)
    kernels.launch_probe_copy(cal, cal.offset(PMC_CAL_BYTES), PMC_CAL_BYTES, stream)
    stream.synchronize()
    del cal

    closed_loop = None
    if args.extras or (not args.skip_kernels and args.workload == "all"):
        # ---- the same step as a closed loop over token ids: embedding lookup in front, the
        # vocabulary projection (151936 x 4096, Q4G128) with the greedy choice fused behind, the
        # chosen tokens being the next step's input.  Reported beside the headline figure, which
        # stays the 36 layers alone.
        vocab = 151936
        hq4 = (rng.integers(0, 256, size=(vocab, hidden // 2), dtype=np.uint8),
               (rng.random((vocab, hidden // 128), np.float32) * 0.004 + 0.004).astype(np.float16),
               (rng.random((vocab, hidden // 128), np.float32) * 2 + 6.5).astype(np.float16))
        head_bufs = [hip.DeviceBuffer.from_numpy(hq4[0]),
                     hip.DeviceBuffer.from_numpy(hq4[1].view(np.uint16)),
                     hip.DeviceBuffer.from_numpy(hq4[2].view(np.uint16))]
        head_bytes = sum(int(a.nbytes) for a in hq4)
        del hq4
        head = kernels.Q4Weight(*[hb.ptr.value for hb in head_bufs])
        d_embed = hip.DeviceBuffer(vocab * hidden * 2)
        d_embed.fill(0x3C)   # every entry the bf16 0x3C3C; the lookup's traffic does not depend on it
        d_tok = hip.DeviceBuffer.from_numpy(rng.integers(0, vocab, size=S, dtype=np.uint32))
        r.cfg.vocab = vocab
        r.ws = hip.DeviceBuffer(kernels.decode_step_workspace_bytes(r.cfg, S, r.num_splits))
        r.batch.token_ids = d_tok.ptr.value
        r.batch.embed_table_bf16 = d_embed.ptr.value
        r.batch.lm_head = C.pointer(head)
        r.batch.out_tokens_u32 = d_tok.ptr.value   # fed back: read by the next step's lookup
        g2 = hip.Graph(stream)
        with g2:
            kernels.launch_pack_ragged(d_ones, d_cur_prior, r.idx["block_tables"],
                                       r.idx["cu_seqlens"], r.slots, r.idx["context_lens"], S, bs,
                                       max_blocks, stream)
            r.launch()
        for i in range(warmup):
            one_step(i, g2)
        stream.synchronize()
        e0.record(stream)
        for i in range(steps):
            one_step(warmup + i, g2)
        e1.record(stream)
        e1.synchronize()
        ms_loop = e0.elapsed_ms(e1) / steps
        toks = d_tok.to_numpy(np.uint32, (S,))
        assert (toks < vocab).all()
        # the vocabulary projection alone (its 330 MB exceed the 256 MB cache: every launch is cold)
        d_xp = hip.DeviceBuffer(kernels.q4_xprep_bytes(S, hidden))
        d_xp.fill(0x3C)
        d_hws = hip.DeviceBuffer(kernels.qgemm_q4g128_greedy_workspace_bytes(S, vocab, hidden))
        d_t2 = hip.DeviceBuffer(S * 4)
        ms_head, _, _ = time_launches(
            stream, [lambda: kernels.launch_qgemm_q4g128_greedy_xprep(
                d_xp, head_bufs[0], head_bufs[1], head_bufs[2], d_t2, None, d_hws, S, vocab, hidden,
                stream)], 40, 4)
        closed_loop = {
            "what": "token ids in, token ids out: embed_lookup + 36 layers + lm_head 151936x4096 "
                    "Q4G128 with greedy fused, chosen tokens fed back on the GPU",
            "ms_per_step": round(ms_loop, 4), "tok_s": round(S / (ms_loop * 1e-3), 1),
            "lm_head_bytes": head_bytes, "lm_head_greedy_us": round(ms_head * 1e3, 1),
            "lm_head_GBps": round(head_bytes / (ms_head * 1e-3) / 1e9, 1)}
        del d_embed, head_bufs
        # leave the runner as it was: 36 layers, hidden state in, hidden state out
        r.cfg.vocab = 0
        r.batch.token_ids = None
        r.batch.lm_head = None

    # ---- the 36 layers over TurboQuant 3-bit KV pools (the reference's KV codec): the fp16
    # pools re-encoded on the device, new rows encoded as the step writes them, attention
    # decoding inside its gather.  A different cache format, so a figure of its own.
    turbo3_step = None
    if args.extras or (not args.skip_kernels and args.workload == "all"):
        rows = r.pools[0][0].nbytes // (hkv * 128 * 2)
        d_iota = hip.DeviceBuffer.from_numpy(np.arange(rows, dtype=np.int64))
        t3_pools = []
        for l in range(L):
            kp, vp = r.pools[l]
            k3, v3 = hip.DeviceBuffer(rows * hkv * 56), hip.DeviceBuffer(rows * hkv * 56)
            kernels.launch_kv_write_turbo3(kp, vp, k3, v3, d_iota, rows, hkv, stream)
            t3_pools.append((k3, v3))
            r.layers[l].k_pool_f16, r.layers[l].v_pool_f16 = k3.ptr.value, v3.ptr.value
        stream.synchronize()
        r.cfg.kv_turbo3 = 1
        g3 = hip.Graph(stream)
        with g3:
            kernels.launch_pack_ragged(d_ones, d_cur_prior, r.idx["block_tables"],
                                       r.idx["cu_seqlens"], r.slots, r.idx["context_lens"], S, bs,
                                       max_blocks, stream)
            r.launch()
        for i in range(warmup):
            one_step(i, g3)
        stream.synchronize()
        e0.record(stream)
        for i in range(steps):
            one_step(warmup + i, g3)
        e1.record(stream)
        e1.synchronize()
        ms_t3 = e0.elapsed_ms(e1) / steps
        out3 = O.bf16_bits_to_f32(r.result_bits())
        assert np.isfinite(out3).all()
        turbo3_step = {
            "what": "the same 36-layer step over TurboQuant 3-bit KV pools (56 bytes per head "
                    "row instead of 256): rows encoded on write, decoded inside the attention",
            "ms_per_step": round(ms_t3, 4), "tok_s": round(S / (ms_t3 * 1e-3), 1),
            "kv_bytes_per_step": int(sum_ctx * L * 2 * hkv * 56)}
        r.cfg.kv_turbo3 = 0
        for l in range(L):
            r.layers[l].k_pool_f16 = r.pools[l][0].ptr.value
            r.layers[l].v_pool_f16 = r.pools[l][1].ptr.value
        del t3_pools

    per_layer_w = sum(int(np.asarray(t[0]).nbytes + np.asarray(t[1]).nbytes +
                          np.asarray(t[2]).nbytes)
                      for t in (layers[0][k] for k in ("qkv", "o", "gate_up", "down")))
    algo_step = L * per_layer_w + sum_ctx * L * 2 * hkv * 128 * 2
    tok_s = S / (ms_step * 1e-3)
    achieved = attn_bytes / (ms_attn * 1e-3) / 1e9
    # hardware-counter traffic of the dominant kernel: the counters cannot be read from inside
    # this process, so the committed summary carries the measured bytes per launch together
    # with the algorithmic bytes of the launches they were measured on (the roofline leg runs
    # at step 0's contexts whatever --steps / --warmup are, so the two agree for this seed)
    traffic = measured_traffic("paged_attn_decode_config5_pmc.txt")
    if measured_traffic("paged_attn_decode_config5_pmc.txt",
                        "algorithmic_bytes_per_launch:") != attn_bytes:
        traffic = None
    return {
        "metric": "decode tok/s @ batch 32 (paged-attn + quant GEMV path)",
        "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "config 5: continuous-batching decode step, Qwen3-8B-style geometry "
                               "(36 layers, hidden 4096, 32 q / 8 kv heads, head_dim 128, MLP "
                               "12288, RMSNorm, RoPE theta 1e6), Q4G128 weights, 32 live sequences, "
                               "contexts U[256,8192], one finishing and one admitted per step, "
                               "fp16 paged KV block 16; embedding and lm_head not included",
                   "mean_sum_ctx": round(sum_ctx, 1), "num_splits": ns,
                   "algorithmic_bytes_per_step": int(algo_step),
                   "step_GBps": round(algo_step / (ms_step * 1e-3) / 1e9, 1),
                   "step_frac_of_hbm_peak": round(algo_step / (ms_step * 1e-3) / 1e9 /
                                                  HBM_PEAK_GBPS, 4),
                   "hip_graph": True, "gpu_side_packing": True},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic,
                     "traffic_source": "profiles/paged_attn_decode_config5_pmc.txt: rocprofv3 "
                                       "--pmc FETCH_SIZE, then WRITE_SIZE, of `bench.py "
                                       "--skip-kernels`, each scaled by what the same counter "
                                       "reads for that command's 256 MiB calibration copy; null "
                                       "when the summary was taken at other bytes per launch",
                     "kernel": "paged_attn_balanced_kernel<4> (decode rows, one layer of the step)",
                     "ms_per_launch": round(ms_attn, 5), "algorithmic_bytes_per_launch": attn_bytes,
                     **against_ceiling(stream, attn_bytes, achieved)},
        "cpu_baseline": {"value": round(S / cpu_s, 3), "unit": "tok/s", "cores": cores,
                         "kind": "port",
                         "sample": f"step 0 in full, 36 layers x 32 sequences, on the CPU oracle "
                                   f"({cpu_s:.1f} s; one layer's weights and pools reused by "
                                   "all 36)"},
        "parity_rel_l2_vs_oracle_one_layer": rel_l2,
        "host_wall_ms_per_step": round(wall_ms, 4),
        "closed_loop_with_embedding_and_lm_head": closed_loop,
        "step_over_turbo3_kv": turbo3_step,
    }


def bench_head_dim64(args):
    """The general-head-width kernel at head_dim 64: config 5's batch at 32 / 8 heads (the
    roofline figure), config 2's batch at Qwen2-0.5B's 14 / 2 heads (checked against the
    oracle), and a mixed batch of two 512-token chunks and six decode rows."""
    import oracle as O
    stream = hip.Stream()

    def timed(case, phases=None):
        r = PagedAttnRunner(case, stream=stream)
        kv_bytes = case["k_pool"].nbytes + case["v_pool"].nbytes
        copies = max(2, min(16, -(-COLD_BYTES // kv_bytes)))
        kps, vps = replicate(r.k_pool, copies), replicate(r.v_pool, copies)
        fns = [lambda k=k, v=v: r.launch(phases=phases, k_pool=k, v_pool=v)
               for k, v in zip(kps, vps)]
        return r, time_launches(stream, fns, args.steps, args.warmup)[0]

    rng = np.random.default_rng(workloads.SEED + 64)
    ctx = rng.integers(256, 8193, size=32)
    big = workloads.paged_case(rng, np.ones(32, np.int32), ctx - 1, hq=32, hkv=8, d=64,
                               pool_period_rows=4099)
    algo = workloads.paged_attn_algorithmic_bytes(big)
    r_big, ms_full = timed(big)
    _, ms_dec = timed(big, kernels.ATTN_PHASE_DECODE)

    ctx = rng.integers(64, 2049, size=16)
    small = workloads.paged_case(rng, np.ones(16, np.int32), ctx - 1, hq=14, hkv=2, d=64)
    r_small, ms_small = timed(small)
    r_small.launch()
    got = r_small.result().astype(np.float32)
    want = O.paged_attn_varlen_fp16(small["q"], small["k_pool"], small["v_pool"],
                                    small["block_tables"], small["cu_seqlens"],
                                    small["context_lens"], 14, 2, 64, small["block_size"],
                                    small["scale"], True).astype(np.float32)
    mixed = workloads.paged_case(rng, [512, 1, 512, 1, 1, 1, 1, 1],
                                 [1000, 3000, 0, 500, 7000, 100, 2000, 4000], hq=32, hkv=8, d=64,
                                 pool_period_rows=4099)
    _, ms_mixed = timed(mixed)
    _, ms_mixed_chunks = timed(mixed, kernels.ATTN_PHASE_PREFILL)
    achieved = algo / (ms_dec * 1e-3) / 1e9

    # a whole decode step at Qwen2-0.5B's geometry (24 layers, hidden 896, 14 q / 2 kv heads of
    # 64, MLP 4864, q/k/v bias), 32 live sequences at fixed contexts U[256,8192]; the layers
    # share one layer's weights (replicated on the device) as the headline step's do
    from tests.gpu_harness import DecodeStepRunner
    S, L = 32, 24
    ctx = rng.integers(256, 8193, size=S)
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=1, hidden=896, hq=14, hkv=2, inter=4864, ctx=ctx, d=64,
        random_nibbles=True, qkv_bias=True, theta=1e4)
    r = DecodeStepRunner(cfg, layers * L, batch, stream=stream, share_layer_data=True)
    ms_model = time_launches(stream, [r.launch], 20, 3)[0]
    kv_bytes_step = int(ctx.sum()) * 2 * 2 * 64 * 2 * L
    w_bytes_layer = sum(w[0].nbytes + w[1].nbytes + w[2].nbytes
                        for w in (layers[0][k] for k in ("qkv", "o", "gate_up", "down")))
    return {
        "metric": "paged-attn decode achieved HBM GB/s (head_dim 64)",
        "value": round(algo / (ms_full * 1e-3) / 1e9, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_full, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "config 5's batch (32 seqs, ctx U[256,8192]) at 32 q / 8 kv heads "
                               "of 64, block 16, fp16 KV: decode + merge",
                   "sum_ctx": int(big["context_lens"].sum()), "num_splits": r_big.num_splits,
                   "algorithmic_bytes_per_step": algo},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "paged_attn_anydim_balanced_kernel<2>",
                     "ms_per_launch": round(ms_dec, 5), **against_ceiling(stream, algo, achieved)},
        "config2_batch_14q_2kv_heads": {"ms_per_step": round(ms_small, 5),
                                        "num_splits": r_small.num_splits,
                                        "algorithmic_bytes_per_step":
                                            workloads.paged_attn_algorithmic_bytes(small),
                                        "parity_max_abs_vs_oracle":
                                            float(np.abs(got - want).max())},
        "mixed_2x512_token_chunks_6_decode_rows": {"ms_per_step": round(ms_mixed, 5),
                                                   "ms_chunk_rows": round(ms_mixed_chunks, 5)},
        "decode_step_qwen2_05b_geometry": {"ms_per_step": round(ms_model, 4),
                                           "tok_s": round(S / (ms_model * 1e-3), 1),
                                           "layers": L, "sum_ctx": int(ctx.sum()),
                                           "num_splits": r.num_splits,
                                           "bytes_per_step": kv_bytes_step + w_bytes_layer * L},
    }


def bench_two_streams(args):
    """Config 5's step as two half-batches of 16 sequences on two equal-priority streams,
    against the one batch of 32 on one stream that the headline times; and, per layer, the
    decode attention of one half on stream A while the other half's chain of projections and
    small operators runs on stream B (fork / join inside one captured graph), against each of
    them alone.  The attention's workers are capped through num_splits (16 x (splits - 1)) to
    leave CUs to the chain.  Weights and pools are shared by the halves."""
    import oracle as O
    from tests.gpu_harness import DecodeStepRunner
    rng = np.random.default_rng(workloads.SEED + 5)
    S, L, hidden, hq, hkv, inter, bs = 32, 36, 4096, 32, 8, 12288, 16
    H = S // 2
    ctx = rng.integers(256, 8193, size=S).astype(np.int64)
    max_ctx = 8194
    cfg, layers, batch = workloads.decode_step_problem(
        rng, num_layers=1, hidden=hidden, hq=hq, hkv=hkv, inter=inter, ctx=np.full(S, max_ctx),
        max_pos=max_ctx + 1, random_nibbles=True)
    max_blocks = batch["block_tables"].shape[1]
    sa, sb = hip.Stream(), hip.Stream()
    prior = (ctx - 1).astype(np.int32)
    cu, slots, ctx_l, _ = O.pack_ragged(np.ones(S, np.int32), prior, batch["block_tables"], bs)
    b0 = dict(batch, h=batch["h"].copy())
    b0.update(cu_seqlens=cu, slots=slots, context_lens=ctx_l, positions=prior)
    r = DecodeStepRunner(cfg, layers * L, b0, stream=sa, share_layer_data=True)
    ev_f, ev_j = hip.Event(), hip.Event()

    def timed(build, n=10, w=3):
        g = hip.Graph(sa)
        with g:
            build()
        for _ in range(w):
            g.launch()
        sa.synchronize()
        e0, e1 = hip.Event(), hip.Event()
        e0.record(sa)
        for _ in range(n):
            g.launch()
        e1.record(sa)
        e1.synchronize()
        return e0.elapsed_ms(e1) / n

    def forked(on_a, on_b):
        ev_f.record(sa)
        sb.wait_event(ev_f)
        on_a()
        on_b()
        ev_j.record(sb)
        sa.wait_event(ev_j)

    # ---- whole steps
    d_cu16 = hip.DeviceBuffer.from_numpy(np.arange(H + 1, dtype=np.int32))

    def half(lo, ns):
        b = kernels.DecodeBatch()
        C.memmove(C.byref(b), C.byref(r.batch), C.sizeof(b))
        b.hidden_f32 = r.h.ptr.value + lo * hidden * 4
        b.out_bf16 = r.out.ptr.value + lo * hidden * 2
        b.block_tables = r.idx["block_tables"].ptr.value + lo * max_blocks * 4
        b.cu_seqlens = d_cu16.ptr.value
        b.context_lens = r.idx["context_lens"].ptr.value + lo * 4
        b.positions = r.idx["positions"].ptr.value + lo * 4
        b.slot_mapping = r.slots.ptr.value + lo * 8
        b.num_seqs, b.num_splits = H, ns
        return b, hip.DeviceBuffer(kernels.decode_step_workspace_bytes(r.cfg, H, ns))

    ms32 = timed(r.launch)
    steps = []
    for ns in (17, 9):
        (ba, wa), (bb, wb) = half(0, ns), half(H, ns)
        step_a = lambda: kernels.launch_decode_step(r.cfg, r.layers, ba, wa, sa)  # noqa: E731
        step_b_on_a = lambda: kernels.launch_decode_step(r.cfg, r.layers, bb, wb, sa)  # noqa: E731
        step_b = lambda: kernels.launch_decode_step(r.cfg, r.layers, bb, wb, sb)  # noqa: E731
        steps.append({"attention_workers": min(256, H * (ns - 1)),
                      "half_alone_ms": round(timed(step_a), 4),
                      "halves_one_after_the_other_ms": round(timed(lambda: (step_a(), step_b_on_a())), 4),
                      "halves_on_two_streams_ms": round(timed(lambda: forked(step_a, step_b)), 4)})

    # ---- per layer: attention of half A beside the chain of half B
    qd, kvd = hq * 128, hkv * 128
    width = qd + 2 * kvd
    d_cu = hip.DeviceBuffer.from_numpy(np.arange(S + 1, dtype=np.int32))
    d_q = hip.DeviceBuffer(S * qd * 2)
    d_q.fill(0x3C)
    xb = lambda k: hip.DeviceBuffer(kernels.q4_xprep_bytes(H, k))  # noqa: E731
    d_attn_b, d_xn, d_act, d_attn_a = xb(qd), xb(hidden), xb(inter), xb(qd)
    for d in (d_attn_b, d_xn, d_act):
        d.fill(0x3C)
    jp = lambda n, k: kernels.qgemm_q4g128_splitk_parts(H, n, k, prepared=True)  # noqa: E731
    j_o, j_gu, j_dn, j_qkv = jp(hidden, qd), jp(2 * inter, hidden), jp(hidden, inter), jp(width, hidden)
    d_proj = hip.DeviceBuffer(max(j_o, j_dn) * H * hidden * 4)
    d_gu = hip.DeviceBuffer(j_gu * H * 2 * inter * 4)
    d_qkv = hip.DeviceBuffer(j_qkv * H * width * 4)
    d_h = hip.DeviceBuffer(H * hidden * 4)
    d_h.fill(0)
    d_q2 = hip.DeviceBuffer(H * qd * 2)
    scale = 1.0 / np.sqrt(128.0)

    def chain(l, stream):
        lay = r.layers[l]
        gemm = lambda x, w, parts, n, k: kernels.launch_qgemm_q4g128_f32_splitk(  # noqa: E731
            x, w.qw, w.scale, w.zero, parts, H, n, k, stream, prepared=True)
        gemm(d_attn_b, lay.o, d_proj, hidden, qd)
        kernels.launch_add_rms_norm_f32p_xprep(d_h, d_proj, j_o, lay.norm2_w_f32, d_xn, H, hidden,
                                               1e-6, stream)
        gemm(d_xn, lay.gate_up, d_gu, 2 * inter, hidden)
        kernels.launch_silu_mul_f32p_xprep(d_gu, j_gu, d_act, H, inter, stream)
        gemm(d_act, lay.down, d_proj, hidden, inter)
        kernels.launch_add_rms_norm_f32p_xprep(d_h, d_proj, j_dn, lay.norm1_w_f32, d_xn, H, hidden,
                                               1e-6, stream)
        gemm(d_xn, lay.qkv, d_qkv, width, hidden)
        kernels.launch_rope_kv_write_f32p(
            d_qkv, j_qkv, r.idx["positions"].ptr.value + H * 4, r.cos, r.sin,
            r.slots.ptr.value + H * 8, d_q2, lay.k_pool_f16, lay.v_pool_f16, H, hq, hkv, 128,
            r.cfg.max_pos, stream)

    us_chain = timed(lambda: [chain(l, sa) for l in range(L)]) * 1e3 / L
    layers_out = []
    for ns in (17, 13, 9):
        ws = hip.DeviceBuffer(kernels.paged_attn_workspace_bytes(H, hq, 128, ns))

        def attn(l, stream):
            lay = r.layers[l]
            kernels.launch_paged_attn_decode_fp16_xprep(
                d_q, lay.k_pool_f16, lay.v_pool_f16, r.idx["block_tables"], d_cu,
                r.idx["context_lens"], d_attn_a, ws, H, hq, hkv, 128, bs, max_blocks, ns, scale,
                stream)
        us_attn = timed(lambda: [attn(l, sa) for l in range(L)]) * 1e3 / L
        us_both = timed(lambda: [forked(lambda l=l: attn(l, sa), lambda l=l: chain(l, sb))
                                 for l in range(L)]) * 1e3 / L
        layers_out.append({"attention_workers": min(256, H * (ns - 1)),
                           "attention_us": round(us_attn, 1), "chain_us": round(us_chain, 1),
                           "both_us": round(us_both, 1),
                           "both_over_sum": round(us_both / (us_attn + us_chain), 3),
                           "both_over_max": round(us_both / max(us_attn, us_chain), 3)})
    return {"workload": "config 5 as two half-batches of 16 sequences on two equal-priority "
                        "streams (36 layers, same weights and pools as the headline step)",
            "one_batch_of_32_on_one_stream_ms": round(ms32, 4), "whole_steps": steps,
            "per_layer_attention_of_one_half_beside_the_chain_of_the_other": layers_out,
            "sum_ctx_half_a": int(ctx[:H].sum()), "sum_ctx_half_b": int(ctx[H:].sum())}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps (default 20 decode steps; 200 launches for the kernel legs)")
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--cpu-seconds", type=float, default=5.0)
    ap.add_argument("--skip-kernels", action="store_true",
                    help="only the decode-step line, without the per-kernel legs")
    ap.add_argument("--extras", action="store_true",
                    help="with --skip-kernels or --workload step: add the two extra legs of the "
                         "decode step (token ids in / token ids out with embedding, lm_head + "
                         "greedy; the step over turbo3 KV pools).  The full default run includes "
                         "both anyway; they are not part of the metric, and runs under a "
                         "profiler leave them out (--skip-kernels without --extras)")
    ap.add_argument("--workload", default="all",
                    choices=["all", "step", "config1", "config2", "config3", "config4",
                             "config4_gemm", "config4_step", "turbo3", "headdim64", "two_streams"],
                    help="all: the decode-step line with every leg inside it (default); "
                         "otherwise only that workload's own JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; every workload is the full single-GPU "
                 "shape and nothing here uses a second device (--gpus must be 1)")
    if hip.device_count() < 1:
        sys.exit("bench.py: no HIP device visible; there is no CPU fallback to time")
    hip.set_device(0)
    kernels.library()
    args.steps_c5 = args.steps if args.steps is not None else 20
    args.warmup_c5 = args.warmup if args.warmup is not None else 3
    if args.workload in ("config1", "config2", "config3", "config4", "config4_gemm",
                         "config4_step", "turbo3", "headdim64", "two_streams"):
        args.steps = args.steps if args.steps is not None else 200
        args.warmup = args.warmup if args.warmup is not None else 20
        leg = {"config1": bench_qgemv_q8, "config2": bench_paged_decode, "config3": bench_q4,
               "config4": bench_mixed_config4, "config4_gemm": bench_q4_tall,
               "config4_step": bench_mixed_step_config4,
               "turbo3": bench_turbo3, "headdim64": bench_head_dim64,
               "two_streams": bench_two_streams}[args.workload]
        print(json.dumps(leg(args)))
        return
    line = bench_decode_step(args)
    if not args.skip_kernels and args.workload == "all":
        args.steps, args.warmup = 200, 20
        c2 = bench_paged_decode(args)
        line["paged_attn_config2"] = {k: c2[k] for k in ("value", "unit", "ms_per_step", "config",
                                                          "roofline", "cpu_baseline",
                                                          "parity_max_abs_vs_oracle")}
        line["mixed_prefill_decode_config4"] = bench_mixed_config4(args)
        line["paged_attn_turbo3_config5"] = bench_turbo3(args)
        line["qgemv_q8_config1"] = bench_qgemv_q8(args)
        line["qgemm_q4_config3"] = bench_q4(args)
        line["qgemm_q4_tall_config4_rows"] = bench_q4_tall(args)
        line["mixed_step_config4_rows"] = bench_mixed_step_config4(args)
        hd = bench_head_dim64(args)
        line["paged_attn_head_dim64"] = {k: hd[k] for k in (
            "value", "unit", "ms_per_step", "config", "roofline", "config2_batch_14q_2kv_heads",
            "mixed_2x512_token_chunks_6_decode_rows", "decode_step_qwen2_05b_geometry")}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
