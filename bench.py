#!/usr/bin/env python3
"""Benchmark of the multi-LoRA apply hot path on one MI355X.

Default run (`python bench.py --gpus 1 --steps K --warmup W`): one JSON line whose headline is the largest
configuration that fits one GPU -- config 5: one decode step of a Llama-2-7B-shaped LoRA path, 32 layers x 7
projections, 1000 rank-32 adapters resident in a paged pool (about 160 GB), 512 decode tokens Zipf(1.1) through
BGMV plus 8 prefill segments of 512 tokens through SGMV in the same step -- and whose `legs` object carries the
other configurations, each timed in the same process on the same device:

    c1  single LoRA-delta op (the CPU reference's case)        c4  prefill SGMV, Llama-13B shapes, bf16
    coldstart  prefill of a request whose adapter is cached / loading (CPU-assisted) / loaded on demand
    c2  decode BGMV, 256 tokens, 64 rank-16 adapters           f1  base projection + LoRA in one pass (c4 batch)
    c3  heterogeneous-rank decode BGMV, 7 projections          reflayout  the reference's own pool layout and call
    maf_trace  a continuous-batching decode sequence driven by the reference's arrival trace and popularity vector

One step of a decode workload = the adapter-pool gather once, then for each layer one BGMV call covering that
layer's projections, accumulating into the base projection outputs; every layer has its own slabs, inputs and
outputs so that a step streams from HBM, not from the 256 MB last-level cache; steps are replayed from a HIP
graph.  `--workload NAME` runs one workload alone and prints its full line.

Every line carries `roofline` (algorithmic bytes or flops of the dominant launches / their measured duration,
HIP events on the launch stream) and the headline carries `cpu_baseline` (the CPU-assisted path's arithmetic on
the host cores, through the package's own CPU library) and `stream_ceiling` (what a plain streaming pass reaches
on this device in this run).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "ae-296_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_BF16_TFLOPS = 2500.0      # dense bf16 / fp16 MFMA peak of the device
MIN_LEG_MS = 100.0                  # every leg is repeated until its timed region is at least this long

# HBM bytes per launch from rocprofv3 counter runs (FETCH_SIZE and WRITE_SIZE, scaled by a copy of known size):
# the figures live in the committed profile summaries, one `key: value` line each, and are read from there.
TRAFFIC_SOURCE = {
    "c2": ("profiles/bgmv_c2_bench.txt", "hbm_bytes_per_decode_call"),
    "c3": ("profiles/bgmv_c3_bench.txt", "hbm_bytes_per_decode_call"),
    "c4": ("profiles/sgmv_c4_bench.txt", "hbm_bytes_per_step"),
    "c5": ("profiles/mixed_c5_bench.txt", "hbm_bytes_per_decode_call"),
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def profile_value(rel_path, key):
    """`key: <number>` from a profile summary under profiles/ (None when the file or the line is absent)."""
    try:
        with open(os.path.join(ROOT, rel_path)) as f:
            for line in f:
                s = line.strip()
                if s.startswith(key + ":"):
                    return float(s.split(":", 1)[1].split()[0])
    except OSError:
        pass
    return None


def traffic_of(workload, applies=True):
    """(traffic, traffic_source) of a roofline object."""
    if workload not in TRAFFIC_SOURCE or not applies:
        return None, None
    path, key = TRAFFIC_SOURCE[workload]
    v = profile_value(path, key)
    return v, (f"{path} ({key}; rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this workload, not this run)"
               if v is not None else f"{path} has no {key} line")


def algorithmic_bytes(T, projs, ranks_of_unique, elt=2):
    """Per projection call: x read + y read and write + every touched adapter's rows once + indices."""
    total = 0
    for hin, hout in projs:
        total += T * hin * elt + 2 * T * hout * elt + int(sum(ranks_of_unique)) * (hin + hout) * elt + 4 * T
    return total


# ---------------------------------------------------------------------------------------------- timing
def percentiles(xs):
    s = sorted(xs)
    pick = lambda q: s[min(len(s) - 1, max(0, int(round(q * (len(s) - 1)))))]
    return {"p10": pick(0.10), "p50": pick(0.50), "p90": pick(0.90)}


def timed(run, reps, warmup):
    """`reps` calls of run() after `warmup` untimed ones, an event after every call on the stream the kernels
    run on.  Returns mean ms per call (first event to last) and the spread of the per-call times."""
    import torch
    for _ in range(warmup):
        run()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(reps):
        run()
        ev[i + 1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    total = ev[0].elapsed_time(ev[reps])
    per = [ev[i].elapsed_time(ev[i + 1]) for i in range(reps)]
    out = {"ms": total / reps, "reps": reps, "timed_ms": total, "wall_s": wall}
    out.update(percentiles(per))
    return out


def reps_for(run, steps, min_ms=MIN_LEG_MS, cap=5000):
    """Repetitions that make the timed region at least min_ms long (never fewer than `steps`)."""
    import torch
    run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3):
        run()
    torch.cuda.synchronize()
    est_ms = max((time.perf_counter() - t0) * 1e3 / 3, 1e-3)
    return int(min(cap, max(steps, math.ceil(min_ms / est_ms))))


def graph_of(fn, enabled=True):
    import torch
    if not enabled:
        return fn
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g.replay


def stream_ceiling(dev):
    """What one plain streaming launch reaches on this device now: nontemporal read of 84 MB and of 1 GB, and an
    in-place read-modify-write of 94 MB and of 1 GB (bytes read + written), rotating over 3 GB so that nothing
    is served by the last-level cache."""
    import torch

    import ctypes

    import mlora
    # the probe kernel lives in a library of its own beside the product one (built by the same Makefile)
    probe = ctypes.CDLL(os.path.join(os.path.dirname(mlora._ext.LIB_PATH), "libmlora_probe.so"))
    probe.mlora_probe_stream.restype = ctypes.c_int
    probe.mlora_probe_stream.argtypes = [ctypes.c_void_p, ctypes.c_longlong, ctypes.c_int, ctypes.c_void_p]
    buf = torch.empty(3 << 30, dtype=torch.uint8, device=dev)
    buf.zero_()
    out = {}
    for name, nbytes, mode in (("read_84MB", 84 << 20, 0), ("read_1GB", 1 << 30, 0), ("rmw_94MB", 47 << 20, 1), ("rmw_1GB", 512 << 20, 1),
                              ("read_with_a_tenth_rewritten_1GB", 1 << 30, 2)):
        n_regions = (3 << 30) // nbytes
        state = {"i": 0}

        def run():
            off = (state["i"] % n_regions) * nbytes
            state["i"] += 1
            rc = probe.mlora_probe_stream(buf.data_ptr() + off, nbytes, mode, mlora._ext.current_stream_ptr())
            if rc:
                raise RuntimeError(f"mlora_probe_stream failed with {rc}")

        # launches back to back between two events (an event per launch would add its own gap to a 13 us launch);
        # best of five such blocks
        n = max(20, min(200, (12 << 30) // nbytes))
        for _ in range(3):
            run()
        best = None
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(n):
                run()
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / n
            best = ms if best is None or ms < best else best
        moved = nbytes * {0: 1.0, 1: 2.0, 2: 1.1}[mode]
        out[name] = {"GBs": moved / (best * 1e-3) / 1e9, "us": best * 1e3, "frac_of_peak": moved / (best * 1e-3) / 1e9 / HBM_PEAK_GBS}
    del buf
    torch.cuda.empty_cache()
    out["note"] = "mean of back-to-back launches (best of five blocks), HIP events; rmw counts bytes read + bytes written"
    return out


# ---------------------------------------------------------------------------------------------- CPU baseline
def host_cores():
    phys = set()
    try:
        pid = cid = None
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("physical id"):
                    pid = line.split(":")[1].strip()
                elif line.startswith("core id"):
                    cid = line.split(":")[1].strip()
                elif not line.strip():
                    if pid is not None and cid is not None:
                        phys.add((pid, cid))
                    pid = cid = None
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    return {"os_cpu_count": os.cpu_count(), "physical_cores": len(phys) or None, "usable_by_this_process": usable}


def cpu_baseline(seconds=3.0):
    """The reference's CPU-assisted LoRA arithmetic (`x.float() @ down @ up -> half`, lora_cpu/lora_shm_op/app.py:136-141,
    one task per request chunk as lora_cpu.py:150-151 shards it) on config 1 -- 32 tokens, 8 rank-16 adapters,
    4096 -> 4096, fp32 weights -- through the package's CPU library (libmlora_cpu.so) on 1 thread and on every
    usable core, and through torch (the library the reference's workers call) on 1 thread and on all."""
    import numpy as np
    import torch

    from mlora import cpu_ops
    rng = np.random.default_rng(1001)
    T, N, r, H = 32, 8, 16, 4096
    down = (rng.standard_normal((N, H, r)) * 0.02).astype(np.float32)
    up = (rng.standard_normal((N, r, H)) * 0.02).astype(np.float32)
    x = rng.standard_normal((T, H)).astype(np.float16).view(np.uint16)
    tok = rng.integers(0, N, T).astype(np.int32)
    host = host_cores()
    all_threads = max(1, min(host["usable_by_this_process"], 64))
    out_buf = np.empty((T, H), np.uint16)

    def port(n_threads):
        pool = cpu_ops.CpuLoraPool(n_threads)
        try:
            cpu_ops.cpu_lora(x, down, up, tok, out=out_buf, tokens_per_task=8, pool=pool)
            n, t0 = 0, time.perf_counter()
            while time.perf_counter() - t0 < seconds:
                cpu_ops.cpu_lora(x, down, up, tok, out=out_buf, tokens_per_task=8, pool=pool)
                n += 1
            dt = time.perf_counter() - t0
        finally:
            pool.close()
        return {"value": T * n / dt, "unit": "token-projections/s", "threads": n_threads, "repetitions": n, "seconds": dt}

    def torch_ref(n_threads):
        prev = torch.get_num_threads()
        try:
            torch.set_num_threads(n_threads)
            xt = torch.from_numpy(x.view(np.float16).copy())
            dn, upt = torch.from_numpy(down), torch.from_numpy(up)
            m, t1 = 0, time.perf_counter()
            while time.perf_counter() - t1 < seconds:
                for t in range(T):
                    a = int(tok[t])
                    (xt[t:t + 1].float() @ dn[a] @ upt[a]).half()
                m += 1
            d1 = time.perf_counter() - t1
        finally:
            torch.set_num_threads(prev)
        return {"value": T * m / d1, "unit": "token-projections/s", "threads": n_threads, "repetitions": m, "seconds": d1}

    p1, pall = port(1), port(all_threads)
    t1, tall = torch_ref(1), torch_ref(all_threads)
    return {"value": pall["value"], "unit": "token-projections/s", "cores": all_threads, "kind": "port",
            "workload": "config 1: single LoRA-delta op on the CPU reference path (not the headline's config 5)",
            "sample": f"config 1 (32 decode tokens, 8 rank-16 adapters, 4096->4096, fp32 weights, one task per token) repeated for "
                      f"{seconds:.0f} s per figure: libmlora_cpu.so on 1 and on {all_threads} persistent worker threads, torch "
                      f"(x.float() @ down @ up -> half per request) on 1 and on {all_threads} threads",
            "host": host, "port_one_thread": p1, "port_all_threads": pall, "torch_one_thread": t1, "torch_all_threads": tall}


def cpu_baseline_prefill(with_base, seconds=10.0):
    """The checker's scalar C on one core over a bounded sample of the config-4 prefill: one segment (128 tokens, or
    32 with the base product) on one rank-64 adapter, q projection 5120 -> 5120, bf16 -- the LoRA delta added
    into y (`with_base` False, the SGMV step) or y = x W + delta (`with_base` True), in TFLOP/s."""
    import numpy as np
    from oracle import oracle as orc
    rng = np.random.default_rng(1004)
    Ts, H, r, page_rows = (32 if with_base else 128), 5120, 64, 8
    n_pages = r // page_rows
    bf = lambda a: orc.to_bits(a.astype(np.float32), orc.BF16)
    x = bf(rng.standard_normal((Ts, H)))
    a_rows = bf(rng.standard_normal((r, H)) * 0.02)
    b_rows = bf(rng.standard_normal((r, H)) * 0.02)
    tbl = np.arange(n_pages, dtype=np.int32)[None, :]
    tok = np.zeros(Ts, np.int32)
    rank, scaling = np.array([r], np.int32), np.array([0.5], np.float32)
    if with_base:
        w = bf(rng.standard_normal((H, H)) / H ** 0.5)
        fn = lambda: orc.gemm_lora_paged(x, w, a_rows, b_rows, tok, tbl, tbl, rank, scaling, page_rows, orc.BF16)
        flops = 2.0 * Ts * H * H + 2.0 * r * 2 * H * Ts
    else:
        y0 = bf(rng.standard_normal((Ts, H)))
        fn = lambda: orc.lora_apply_paged(x, a_rows, b_rows, tok, tbl, tbl, rank, scaling, page_rows, orc.BF16, y0=y0)
        flops = 2.0 * r * 2 * H * Ts
    fn()
    n, t0 = 0, time.perf_counter()
    while n == 0 or time.perf_counter() - t0 < seconds:
        fn()
        n += 1
    dt = time.perf_counter() - t0
    return {"value": flops * n / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": f"one {Ts}-token segment, one rank-64 adapter, q projection 5120->5120, bf16"
                      f"{', with the base product' if with_base else ''}: {n} repetitions in {dt:.1f} s on one core"}


# ---------------------------------------------------------------------------------------------- prefill workloads
def _c4_batch(dev, with_weights):
    import numpy as np
    import torch

    import mlora
    from mlora import workloads
    rng = np.random.default_rng(1004)
    lens = rng.integers(128, 1025, 16).astype(np.int32)
    adapters = rng.integers(0, 32, 16).astype(np.int32)
    starts = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    T = int(lens.sum())
    projections = workloads.LLAMA13B_ALL
    pool = mlora.AdapterPool(1, projections, 32, 32 * 8, page_rows=8, max_rank=64, dtype=torch.bfloat16, device=dev)
    workloads.fill_pool(pool, np.full(32, 64, np.int32), np.full(32, 0.5, np.float32), rng, seed=1004)
    seg = tuple(torch.from_numpy(a).to(dev) for a in (starts, lens, adapters))
    gen = torch.Generator(device=dev)
    gen.manual_seed(4004)
    x = {h: torch.randn(T, h, device=dev, generator=gen).bfloat16() for h in (5120, 13824)}
    y = {p: torch.randn(T, projections[p][1], device=dev, generator=gen).bfloat16() for p in projections}
    # q, k, v read the attention input, gate and up the MLP input; o and down have inputs of their own
    x_o = torch.randn(T, 5120, device=dev, generator=gen).bfloat16()
    x_ffn = torch.randn(T, 5120, device=dev, generator=gen).bfloat16()
    x_in = {"q": x[5120], "k": x[5120], "v": x[5120], "o": x_o, "gate": x_ffn, "up": x_ffn, "down": x[13824]}
    w = None
    if with_weights:
        w = {p: (torch.randn(projections[p], device=dev, generator=gen) / projections[p][0] ** 0.5).bfloat16() for p in projections}
    ws = mlora.sgmv_workspace(T, 16, dev, n_proj=len(projections))
    return dict(T=T, projections=projections, pool=pool, seg=seg, adapters=adapters, x=x, y=y, x_in=x_in, w=w, ws=ws,
                names=list(projections))


def bench_c4(args, dev, steps, warmup, min_ms=0.0, cpu=True):
    """Prefill SGMV, config 4: Llama-13B shapes (hidden 5120, MLP 13824), 16 requests with prompt lengths
    U[128, 1024], each bound to one of 32 rank-64 adapters, bf16, tokens packed per request.  One step =
    the plan once, then the seven projections of one layer (q, k, v, o, gate, up, down) in one call."""
    import numpy as np

    import mlora
    b = _c4_batch(dev, False)
    T, projections, pool, names, y, x, x_in = b["T"], b["projections"], b["pool"], b["names"], b["y"], b["x"], b["x_in"]

    def step():
        plan = mlora.plan_prefill(*b["seg"], T, pool, workspace=b["ws"])      # once per batch, shared by the projections
        if args.fused:                                                        # one call per projection (3 launches each)
            for p, (hin, hout) in projections.items():
                mlora.sgmv(y[p], x[hin], pool, 0, p, accumulate=True, plan=plan)
        else:                                                                 # all seven in one call (3 launches)
            mlora.sgmv_multi([y[p] for p in names], [x_in[p] for p in names], pool, 0, names, plan)

    reps = reps_for(step, steps, min_ms) if min_ms else steps
    t = timed(step, reps, warmup)
    ms_per_step = t["ms"]
    flops = sum(2.0 * 64 * (hin + hout) * T for hin, hout in projections.values())
    uniq = np.unique(b["adapters"])
    alg = sum(T * hin * 2 + 2 * T * hout * 2 + len(uniq) * 64 * (hin + hout) * 2 + 4 * T + 12 * 16
              for hin, hout in projections.values())
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    gbs = alg / (ms_per_step * 1e-3) / 1e9
    traffic, src = traffic_of("c4", not args.fused)
    return {"metric": "SGMV prefill throughput", "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": reps,
            "warmup": warmup, "ms_per_step": ms_per_step, "ms_per_step_spread": {k: t[k] for k in ("p10", "p50", "p90")},
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "config 4: prefill SGMV, Llama-13B q/k/v/o/gate/up/down, 16 requests U[128,1024], "
                                   "32 rank-64 adapters, bf16", "tokens": T, "segments": 16,
                       "form": "one call per projection" if args.fused else "one call over the 7 projections"},
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                         "traffic": traffic, "traffic_source": src,
                         "kernel": "sgmv plan (once) + 7 x (shrink, reduce, expand)" if args.fused else
                                   "sgmv plan (once) + one shrink, reduce and expand launch over the 7 projections",
                         "algorithmic_bytes_per_step": alg, "flops_per_step": flops, "mfma_tflops": tflops,
                         "mfma_frac": tflops / MFMA_PEAK_BF16_TFLOPS,
                         "mfma_frac_ceiling": (flops / alg) / (MFMA_PEAK_BF16_TFLOPS * 1e12 / (HBM_PEAK_GBS * 1e9))},
            "cpu_baseline": cpu_baseline_prefill(False) if cpu else None}


def bench_f1(args, dev, steps, warmup, min_ms=0.0, cpu=True):
    """Base projection + LoRA in one pass on the config-4 batch (Llama-13B shapes, 16 requests U[128, 1024],
    32 rank-64 adapters, bf16): one step = q, k, v, o, gate, up, down of one layer, y = x W + delta, as one
    mlora_gemm_lora_planned call (shrink, scaled reduce, one GEMM launch).  The same step as the reference runs
    it -- library GEMM per projection, then the SGMV kernels adding the delta -- is timed beside it."""
    import torch

    import mlora
    b = _c4_batch(dev, True)
    T, projections, pool, names, x_in, w = b["T"], b["projections"], b["pool"], b["names"], b["x_in"], b["w"]
    y = {p: torch.empty(T, projections[p][1], device=dev, dtype=torch.bfloat16) for p in names}

    def fused():
        plan = mlora.plan_prefill(*b["seg"], T, pool, workspace=b["ws"], aligned=True)
        mlora.gemm_lora([y[p] for p in names], [x_in[p] for p in names], [w[p] for p in names], pool, 0, names, plan)

    def unfused():
        plan = mlora.plan_prefill(*b["seg"], T, pool, workspace=b["ws"])
        for p in names:
            torch.mm(x_in[p], w[p], out=y[p])
        mlora.sgmv_multi([y[p] for p in names], [x_in[p] for p in names], pool, 0, names, plan)

    def base_only():
        for p in names:
            torch.mm(x_in[p], w[p], out=y[p])

    reps = reps_for(fused, steps, min_ms) if min_ms else steps
    side = max(5, min(reps, steps))
    ms_unfused = timed(unfused, side, warmup)["ms"]
    ms_base = timed(base_only, side, warmup)["ms"]
    t = timed(fused, reps, warmup)
    ms_per_step = t["ms"]
    flops = sum(2.0 * T * hin * hout + 2.0 * 64 * (hin + hout) * T for hin, hout in projections.values())
    # every operand once: x, W, y written, the touched adapters' rows
    hbm_bytes = sum(T * hin * 2 + hin * hout * 2 + T * hout * 2 for hin, hout in projections.values())
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    return {"metric": "base projection + LoRA prefill throughput", "value": tflops, "unit": "TFLOP/s", "n_gpus": 1,
            "steps": reps, "warmup": warmup, "ms_per_step": ms_per_step,
            "ms_per_step_spread": {k: t[k] for k in ("p10", "p50", "p90")}, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "config-4 batch with base weights: Llama-13B q/k/v/o/gate/up/down, 16 requests U[128,1024], "
                                   "32 rank-64 adapters, bf16; y = x W + delta in one pass", "tokens": T, "segments": 16,
                       "form": "shrink + scaled reduce + one GEMM launch over the 7 projections",
                       "library_gemm_then_sgmv_ms": ms_unfused, "library_gemm_alone_ms": ms_base,
                       "speedup_over_library_gemm_then_sgmv": ms_unfused / ms_per_step},
            "roofline": {"bound": "mfma", "achieved": tflops, "peak": MFMA_PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": tflops / MFMA_PEAK_BF16_TFLOPS, "traffic": None, "traffic_source": None,
                         "kernel": "sgmv shrink + scaled reduce + gemm_lora_kernel (one launch over the 7 projections)",
                         "flops_per_step": flops, "mfma_frac": tflops / MFMA_PEAK_BF16_TFLOPS,
                         "hbm_frac": hbm_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, "operand_bytes_per_step": hbm_bytes},
            "cpu_baseline": cpu_baseline_prefill(True) if cpu else None}


# ---------------------------------------------------------------------------------------------- reference layout
def bench_reflayout(args, dev, steps, warmup, min_ms=0.0):
    """The reference's own decode call on its own pool layout (lora_gpu.py:33-40,122-163) at config-2 size: q, k, v
    of one layer, pool tensors [N, L, r, Hin] / [N, L, Hout, r], int64 indices, y = zeros then y += delta
    (`Lora_GPU.invoke_one_layer_{q,k,v}`), 32 layers per step, eager as the reference calls it and from a HIP graph."""
    import numpy as np
    import torch

    import mlora
    from mlora import workloads
    T, N, L, r, H = 256, 64, 32, 16, 4096
    rng = np.random.default_rng(1002)
    cfg = dict(n_layers=L, batch_size=N, lora_rank=r, hidden_dim=H, tp_degree=1, max_prefill_batch_size=1)
    gpu = mlora.Lora_GPU(cfg, device=dev, seed=7)
    ids = torch.from_numpy(workloads.zipf_adapters(rng, T, N, 1.0).astype(np.int64)).to(dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(2002)
    xs = [torch.randn(T, H, device=dev, generator=gen).half() for _ in range(L)]

    batched = getattr(gpu, "invoke_one_layer_qkv", None) if not args.fused else None    # --fused: one call per projection

    def step():
        if batched is not None:
            gpu.plan_decode(T, ids)                          # once per step, as a serving loop would
        for l in range(L):
            if batched is not None:
                batched(xs[l], l, lora_ids=ids)
            else:
                for f in (gpu.invoke_one_layer_q, gpu.invoke_one_layer_k, gpu.invoke_one_layer_v):
                    f(xs[l], l, False, lora_ids=ids)

    step()
    torch.cuda.synchronize()
    reps = reps_for(step, steps, min_ms) if min_ms else steps
    eager = timed(step, reps, warmup)
    # under a graph the output buffers are those of the capture
    run = graph_of(step)
    greps = reps_for(run, steps, min_ms) if min_ms else steps
    t = timed(run, greps, warmup)
    # the paged call on the same batch (same index vector, q/k/v, rank-16 adapters on pool pages), for the ratio
    wl = workloads.make_decode("ref_cmp", {p: (H, H) for p in "qkv"}, L, T, N, [r], 1.0, seed=1002, device=dev,
                               tok_adapter=ids.cpu().numpy().astype(np.int32))
    tok32 = torch.from_numpy(wl.tok_adapter).to(dev)
    pplan = mlora.plan_decode(tok32, wl.pool, group=4)
    pys = [[torch.empty(T, H, device=dev, dtype=torch.float16) for _ in range(3)] for _ in range(L)]

    def paged_step():
        mlora.plan_decode(tok32, wl.pool, group=4, out=pplan)
        for l in range(L):
            mlora.bgmv(pys[l], [xs[l]] * 3, wl.pool, l, ["q", "k", "v"], tok32, plan=pplan, accumulate=False, fused=False)

    paged_step()
    torch.cuda.synchronize()
    prun = graph_of(paged_step)
    tp = timed(prun, reps_for(prun, steps, min_ms) if min_ms else steps, warmup)
    del wl, pplan, pys
    uniq = np.unique(ids.cpu().numpy())
    # x is read once for q, k, v; y is written, not read (the call starts from zeros); indices are int64
    alg = T * H * 2 + 3 * T * H * 2 + 3 * len(uniq) * r * (H + H) * 2 + 8 * T
    launch_us = t["ms"] * 1e3 / L
    achieved = alg / (launch_us * 1e-6) / 1e9
    return {"metric": "BGMV decode throughput on the reference's pool layout", "value": T * 3 * L / (t["ms"] * 1e-3),
            "unit": "token-projections/s", "n_gpus": 1, "steps": greps, "warmup": warmup, "ms_per_step": t["ms"],
            "ms_per_step_spread": {k: t[k] for k in ("p10", "p50", "p90")}, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": "reference layout, config-2 size: q/k/v 4096->4096, 256 tokens, 64 rank-16 adapters, Zipf(1.0), "
                                   "fp16, pool [N,L,r,Hin] / [N,L,Hout,r], int64 indices", "layers": L, "tokens": T,
                       "form": "one q/k/v call per layer" if batched is not None else "one call per projection", "hip_graph": True,
                       "eager_ms_per_step": eager["ms"], "eager_spread": {k: eager[k] for k in ("p10", "p50", "p90")},
                       "paged_call_same_batch_ms_per_step": tp["ms"], "ratio_to_paged_call": t["ms"] / tp["ms"]},
            "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                         "traffic": None, "traffic_source": None, "kernel": "one layer's q/k/v calls on the reference layout",
                         "launch_us": launch_us, "algorithmic_bytes_per_launch": alg},
            "cpu_baseline": None}


# ---------------------------------------------------------------------------------------------- swap-in, transport
def bench_swap(args, dev):
    """Adapter swap-in (cold start): one rank-64 adapter for q/k/v of a 32-layer, hidden-4096 model (the shape the
    reference's swapper is started with, shared_tensor.py:23-30) from pinned host memory onto its pool pages.
    One step = one whole adapter.  Beside it, the copy pattern of the reference's swapper restated with torch
    (per layer and tensor a pageable host->device copy and a slice assignment, shared_tensor.py:117-147)."""
    import torch

    import mlora
    L, H, r = 32, 4096, 64
    projections = {p: (H, H) for p in "qkv"}
    pool = mlora.AdapterPool(L, projections, n_slots=4, n_pages=64, page_rows=8, max_rank=r, dtype=torch.float16, device=dev)
    loader = mlora.AdapterLoader(pool, layers_per_copy=args.layers if args.layers > 0 else 8, first_layer=8)
    gen = torch.Generator().manual_seed(3003)
    w = {p: (torch.randn(L, H, r, generator=gen) * 0.001, torch.randn(L, r, H, generator=gen) * 0.001) for p in "qkv"}
    host = loader.stage(w, r, 0.5)
    nbytes = host.nbytes

    def one(slot):
        t0 = time.perf_counter()
        ticket = loader.load_async(slot, host)
        t_issue = time.perf_counter() - t0
        first = None
        while not ticket.ready(15):                      # the reference's progress code 2: layers 8..15 are in
            pass
        first = time.perf_counter() - t0
        ticket.wait()
        return t_issue, first, time.perf_counter() - t0

    for i in range(args.warmup):
        one(i % 4)
    res = [one(i % 4) for i in range(args.steps)]
    torch.cuda.synchronize()
    issue = sum(r_[0] for r_ in res) / len(res)
    first = sum(r_[1] for r_ in res) / len(res)
    total = sum(r_[2] for r_ in res) / len(res)

    # the reference's copy pattern on the same box (torch restatement, not the reference's code)
    dense = [torch.empty((4, L, r, H), dtype=torch.float16, device=dev) for _ in range(6)]
    cpu_down = [(0.001 * torch.randn(H, r)).half().t().contiguous() for _ in range(L)]
    cpu_up = [(0.001 * torch.randn(r, H)).half().t().contiguous() for _ in range(L)]

    def ref_style(j):
        t0 = time.perf_counter()
        for k in list(range(8, L)) + list(range(0, 8)):
            for i in range(3):
                dense[i][j, k] = cpu_up[k].to(dev).t()
            for i in range(3, 6):
                dense[i][j, k] = cpu_down[k].to(dev)
            if k in (15, 23, 31):
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    ref_style(0)
    n_ref = max(3, args.steps // 5)
    ref_t = sum(ref_style(i % 4) for i in range(n_ref)) / n_ref

    gbs = nbytes / total / 1e9
    return {"metric": "adapter swap-in throughput (host pinned -> pool pages)", "value": gbs, "unit": "GB/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": total * 1e3,
            "ms_per_step_spread": percentiles([r_[2] * 1e3 for r_ in res]), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "u16", "data": "synthetic",
            "config": {"workload": "swap-in of one rank-64 adapter, q/k/v, 32 layers, hidden 4096, fp16",
                       "bytes_per_adapter": nbytes, "layers_per_copy": loader.layers_per_copy,
                       "ms_until_layers_8_15_ready": first * 1e3, "ms_host_time_to_issue": issue * 1e3},
            "roofline": {"bound": "pcie", "achieved": gbs, "peak": 64.0, "unit": "GB/s", "frac": gbs / 64.0, "traffic": None,
                         "traffic_source": None, "kernel": "host->device copies (copy engine) + scatter_kernel"},
            "cpu_baseline": {"value": nbytes / ref_t / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                             "sample": f"the swapper's copy pattern (pageable host tensors, one copy and one slice assignment per "
                                       f"layer and tensor) restated with torch, {n_ref} adapters, {ref_t * 1e3:.2f} ms each"}}


def bench_assist(args, dev):
    """CPU-assisted prefill of the reference's shape (hidden 4096, slots of 256 tokens, 64 tokens per worker; 8 requests
    of 256 tokens): hidden states to the host request slots plus the wake-up codes, the q/k/v chunks on the package's
    in-process workers (libmlora_cpu.so), and the result slots back to the device.  The transport alone is timed with
    the signals cleared by hand.  Beside it, the reference's call pattern restated with torch (one device->host copy
    per request, one host->device copy per finished chunk and projection, lora_cpu.py:176-232)."""
    import numpy as np
    import torch

    import mlora
    B, tkn, H, cap, r = 8, 256, 4096, 64, 16
    cfg = dict(batch_size=B, lora_num=64, tp_degree=1, hidden_dim=H, lora_rank=r, token_per_lora=cap, n_layers=32)
    cpu = mlora.Lora_CPU(cfg, gpu_id=0, device=dev)
    hidden = torch.randn(B * tkn, H, device=dev).half()
    e = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    t_exp = t_imp = 0.0
    for i in range(args.warmup + args.steps):
        e[0].record()
        cpu.invoke_lora_async(hidden, tkn)
        e[1].record()
        torch.cuda.synchronize()
        cpu.np_signal[:] = 0                                   # the workers' part: nothing computed here
        e[2].record()
        cpu.collect_qkv(tkn, B)
        e[3].record()
        torch.cuda.synchronize()
        if i >= args.warmup:
            t_exp += e[0].elapsed_time(e[1])
            t_imp += e[2].elapsed_time(e[3])
    t_exp, t_imp = t_exp / args.steps, t_imp / args.steps
    b_exp, b_imp = B * tkn * H * 2, 3 * B * tkn * H * 2

    # the whole CPU-assisted call with the in-process workers: export -> 3 x 32 chunks of 64 tokens on the host cores -> import
    rng = np.random.default_rng(77)
    down = [(rng.standard_normal((1, H, r)) * 0.001).astype(np.float32) for _ in range(3)]
    up = [(rng.standard_normal((1, r, H)) * 0.001).astype(np.float32) for _ in range(3)]
    n_threads = max(1, min(host_cores()["usable_by_this_process"], 64))
    cpu.start_workers(down, up, n_threads=n_threads)
    whole = []
    for i in range(3 + max(3, args.steps // 4)):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        cpu.invoke_lora_async(hidden, tkn)
        cpu.collect_qkv(tkn, B)
        torch.cuda.synchronize()
        if i >= 3:
            whole.append((time.perf_counter() - t0) * 1e3)
    cpu.stop_workers()

    # reference call pattern, restated: pinned host tensors, one copy per request out, one per chunk back
    slots = torch.empty((64, 256, H), dtype=torch.float16, pin_memory=True)
    outs = [torch.empty((64, 256, H), dtype=torch.float16, pin_memory=True) for _ in range(3)]
    res = [torch.empty((B, tkn, H), dtype=torch.float16, device=dev) for _ in range(3)]
    hv = hidden.view(B, tkn, H)
    cpr = (tkn - 1) // cap + 1

    def ref_style():
        t0 = time.perf_counter()
        for b in range(B):
            slots[b, :tkn].copy_(hv[b], non_blocking=True)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for q in range(3):
            for b in range(B):
                for o in range(cpr):
                    res[q][b, o * cap:(o + 1) * cap].copy_(outs[q][b, o * cap:(o + 1) * cap])      # synchronous, as cudaHtoD2D is
        torch.cuda.synchronize()
        return t1 - t0, time.perf_counter() - t1

    ref_style()
    rr = [ref_style() for _ in range(max(3, args.steps // 5))]
    r_exp, r_imp = sum(x[0] for x in rr) / len(rr) * 1e3, sum(x[1] for x in rr) / len(rr) * 1e3
    cpu.close()
    gbs = (b_exp + b_imp) / ((t_exp + t_imp) * 1e-3) / 1e9
    return {"metric": "CPU-assist transport throughput (device <-> pinned host slots)", "value": gbs, "unit": "GB/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": t_exp + t_imp, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "u16", "data": "synthetic",
            "config": {"workload": "8 requests x 256 tokens, hidden 4096: export 16.8 MB + wake-up codes, import q/k/v 50.3 MB",
                       "export_ms": t_exp, "import_ms": t_imp, "export_GBs": b_exp / t_exp / 1e6, "import_GBs": b_imp / t_imp / 1e6,
                       "whole_call_with_in_process_workers_ms": percentiles(whole), "worker_threads": n_threads},
            "roofline": {"bound": "pcie", "achieved": gbs, "peak": 64.0, "unit": "GB/s", "frac": gbs / 64.0, "traffic": None,
                         "traffic_source": None, "kernel": "assist_export_kernel + assist_signal_kernel, assist_import_kernel"},
            "cpu_baseline": {"value": (b_exp + b_imp) / ((r_exp + r_imp) * 1e-3) / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                             "sample": f"the reference's call pattern restated with torch: {B} copies out ({r_exp:.3f} ms), "
                                       f"{3 * B * cpr} synchronous chunk copies back ({r_imp:.3f} ms)"}}


# ---------------------------------------------------------------------------------------------- decode workloads
# `inputs` names the activation tensor each projection reads (projections that read the same tensor in the
# model share it here).  `layers` is chosen so that a step's working set is far larger than the 256 MB
# last-level cache.
_IN = {"q": "attn", "k": "attn", "v": "attn", "o": "o", "gate": "ffn", "up": "ffn", "down": "down"}
DECODE = {
    "c1": dict(desc="config 1: single LoRA-delta op, q_proj 4096->4096, 32 decode tokens, 8 rank-16 adapters, "
                    "uniform adapter per token, fp16, scaling 2.0",
               projs=["q"], shapes="7b_attn", T=32, N=8, ranks=[16], alpha=0.0, layers=256, seed=1001),
    "c2": dict(desc="config 2: decode BGMV, Llama-7B q/k/v/o 4096->4096, 256 tokens, 64 rank-16 adapters, "
                    "Zipf(1.0), fp16, scaling 2.0",
               projs=["q", "k", "v", "o"], shapes="7b_attn", T=256, N=64, ranks=[16], alpha=1.0, layers=32, seed=1002),
    "c3": dict(desc="config 3: heterogeneous-rank decode BGMV, 128 adapters with ranks from {8,16,32,64} in a paged "
                    "pool, Llama-7B q/k/v/o, gate/up, down, 128 tokens, Zipf(1.2), fp16, scaling 32/r",
               projs=["q", "k", "v", "o", "gate", "up", "down"], shapes="7b_all", T=128, N=128, ranks=None, alpha=1.2,
               layers=4, seed=1003),
    "c5": dict(desc="config 5: one decode step of a Llama-2-7B-shaped LoRA path, 32 layers x 7 projections, 1000 rank-32 "
                    "adapters resident in a paged pool, 512 decode tokens Zipf(1.1), plus 8 prefill segments of 512 "
                    "tokens through SGMV in the same step, fp16",
               projs=["q", "k", "v", "o", "gate", "up", "down"], shapes="7b_all", T=512, N=1000, ranks=[32], alpha=1.1,
               layers=32, seed=1005, prefill=(8, 512)),
}
# Decode batches whose adapter ids are drawn from the reference's measured adapter-popularity vectors
# (benchmark/maf_lora_popularity/popularity_{128,256,512}.npy, kept as data under tests/golden/) the way its
# load generator draws them (benchmark/client_maf.py:41-42,53); q/k/v only, as the reference applies LoRA.
for _n in (128, 256, 512):
    DECODE[f"maf{_n}"] = dict(
        desc=f"decode BGMV, Llama-7B q/k/v 4096->4096, 256 running requests, {_n} rank-16 adapters, adapter per "
             f"request from the reference's popularity_{_n}.npy, fp16, scaling 2.0",
        projs=["q", "k", "v"], shapes="7b_attn", T=256, N=_n, ranks=[16], alpha=0.0, layers=32, seed=2000 + _n,
        popularity=os.path.join(ROOT, "tests", "golden", f"maf_popularity_{_n}.npy"))


def bench_decode(args, dev, workload, steps, warmup, min_ms=0.0):
    """One decode workload: its full JSON line.  With min_ms > 0 the step is repeated until the timed region is that
    long (legs); otherwise exactly `steps` steps are timed."""
    import numpy as np
    import torch

    import mlora
    from mlora import workloads

    cfg = DECODE[workload]
    group = args.group if args.group >= 0 else mlora.ops.group_for(cfg["T"], len(cfg["projs"]), cfg["N"])
    L = args.layers if args.layers > 0 else cfg["layers"]
    shapes = workloads.LLAMA7B_ATTN if cfg["shapes"] == "7b_attn" else workloads.LLAMA7B_ALL
    projs = cfg["projs"]
    shapes = {p: shapes[p] for p in projs}
    rng = np.random.default_rng(cfg["seed"])
    ranks = cfg["ranks"] if cfg["ranks"] is not None else rng.choice([8, 16, 32, 64], size=cfg["N"]).astype(np.int32)
    log(f"building {workload} with {L} layers ...")
    lora_ids = None
    if cfg.get("popularity"):
        lora_ids = workloads.draw_lora_ids(np.load(cfg["popularity"], allow_pickle=False), cfg["T"], seed=0)
    wl = workloads.make_decode(workload, shapes, L, cfg["T"], cfg["N"], ranks, cfg["alpha"], seed=cfg["seed"],
                               device=dev, alpha_lora=32.0, tok_adapter=lora_ids)
    pool, T = wl.pool, len(wl.tok_adapter)
    log(f"pool slabs: {sum(t.numel() * 2 for t in list(pool.a_rows.values()) + list(pool.b_rows.values())) / 1e9:.2f} GB")
    tok = torch.from_numpy(wl.tok_adapter).to(dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(cfg["seed"] + 1000)
    inputs = sorted({_IN[p] for p in projs})
    width = {_IN[p]: shapes[p][0] for p in projs}
    xs = [{i: torch.randn(T, width[i], device=dev, generator=gen).half() for i in inputs} for _ in range(L)]
    ys = [[torch.randn(T, shapes[p][1], device=dev, generator=gen).half() for p in projs] for _ in range(L)]
    plan = mlora.plan_decode(tok, pool, group=group) if group else None
    fused = bool(args.fused or plan is None or
                 (not args.split and mlora.ops.decode_fused(T, group, len(projs), pool.n_slots)))

    # config 5 carries prefill segments through SGMV in the same step (activations shared by the layers:
    # they are larger than the last-level cache anyway)
    pre = None
    if cfg.get("prefill"):
        n_seg, seg_len = cfg["prefill"]
        Tp = n_seg * seg_len
        seg_adapter = workloads.zipf_adapters(rng, n_seg, cfg["N"], cfg["alpha"])
        ss = torch.arange(0, Tp, seg_len, dtype=torch.int32, device=dev)
        sl = torch.full((n_seg,), seg_len, dtype=torch.int32, device=dev)
        sa = torch.from_numpy(seg_adapter).to(dev)
        px = {i: torch.randn(Tp, width[i], device=dev, generator=gen).half() for i in inputs}
        py = {p: torch.randn(Tp, shapes[p][1], device=dev, generator=gen).half() for p in projs}
        pre = dict(ss=ss, sl=sl, sa=sa, T=Tp, x=px, y=py, ws=mlora.sgmv_workspace(Tp, n_seg, dev, n_proj=len(projs)),
                   adapters=seg_adapter)

    side = mlora.SideStream(dev) if (pre is not None and not args.one_stream) else None

    def bgmv_layers():
        for l in range(L):
            mlora.bgmv(ys[l], [xs[l][_IN[p]] for p in projs], pool, l, projs, tok, plan=plan, fused=fused)

    def step():
        if plan is not None:
            mlora.plan_decode(tok, pool, group=group, out=plan)
        if pre is None:
            bgmv_layers()
            return
        pplan = mlora.plan_prefill(pre["ss"], pre["sl"], pre["sa"], pre["T"], pool, workspace=pre["ws"])
        for l in range(L):
            def decode_half(l=l):
                mlora.bgmv(ys[l], [xs[l][_IN[p]] for p in projs], pool, l, projs, tok, plan=plan, fused=fused)

            def prefill_half(l=l):
                mlora.sgmv_multi([pre["y"][p] for p in projs], [pre["x"][_IN[p]] for p in projs], pool, l, projs, pplan)

            if side is None:
                decode_half()
                prefill_half()
            else:
                # the two halves of a layer run side by side and are joined before the next layer starts
                mlora.side_by_side(side, prefill_half, decode_half)

    step()
    torch.cuda.synchronize()
    run_step = graph_of(step, not args.no_graph)
    reps = reps_for(run_step, steps, min_ms) if min_ms else steps
    t = timed(run_step, reps, warmup)
    ms_per_step = t["ms"]
    n_tok = T + (pre["T"] if pre else 0)
    value = n_tok * len(projs) * L / (ms_per_step * 1e-3)

    uniq = np.unique(wl.tok_adapter[wl.tok_adapter >= 0])
    shp = [shapes[p] for p in projs]
    alg = algorithmic_bytes(T, shp, wl.ranks[uniq])
    per_token_gather = sum(T * h[0] * 2 + 2 * T * h[1] * 2 + int(wl.ranks[wl.tok_adapter].sum()) * (h[0] + h[1]) * 2 + 4 * T
                           for h in shp)
    # The BGMV calls alone (the same layers without gather, plan and prefill launches): the roofline figure.
    run_bgmv = graph_of(bgmv_layers, not args.no_graph)
    tk = timed(run_bgmv, reps_for(run_bgmv, steps, min_ms) if min_ms else steps, warmup)
    launch_us = tk["ms"] * 1e3 / L
    achieved = alg / (launch_us * 1e-6) / 1e9
    kernel = ("bgmv_kernel" if fused else "bgmv_shrink_kernel + bgmv_expand_kernel (one layer's pair)") + \
             f", {len(projs)} projections per call"
    extra = {"launch_us": launch_us, "launch_us_spread": {k: tk[k] * 1e3 / L for k in ("p10", "p50", "p90")},
             "algorithmic_bytes_per_launch": alg, "per_token_gather_bytes_per_launch": per_token_gather}
    if pre is not None:
        # Mixed step: decode and prefill bytes of all layers over the whole step (gather and plan included).
        pu = np.unique(pre["adapters"])
        alg_pre = algorithmic_bytes(pre["T"], shp, wl.ranks[pu]) + 12 * len(pre["adapters"]) * len(projs)
        alg_step = (alg + alg_pre) * L
        extra.update({"whole_step": {"achieved": alg_step / (ms_per_step * 1e-3) / 1e9,
                                     "frac": alg_step / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                     "algorithmic_bytes_per_step": alg_step, "prefill_bytes_per_layer": alg_pre,
                                     "kernels": "gather + prefill plan + 32 x (decode pair + SGMV shrink, reduce, expand over 7 projections)"}})
    traffic, src = traffic_of(workload, group == mlora.ops.group_for(cfg["T"], len(projs), cfg["N"]) and L == cfg["layers"] and not fused)

    metric = "BGMV decode throughput (LoRA-applied token-projections per second)"
    if pre is not None:
        metric = (f"multi-LoRA apply throughput of the mixed step ({T} decode tokens through BGMV + {pre['T']} prefill tokens "
                  "through SGMV, LoRA-applied token-projections per second)")
    out = {
        "metric": metric,
        "value": value, "unit": "token-projections/s", "n_gpus": 1, "steps": reps, "warmup": warmup,
        "ms_per_step": ms_per_step, "ms_per_step_spread": {k: t[k] for k in ("p10", "p50", "p90")},
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": cfg["desc"], "layers": L, "projections_per_call": len(projs),
                   "launches_per_step": L * (1 if fused else 2) + (1 if plan else 0) + ((1 + 3 * L) if pre else 0),
                   "form": "fused" if fused else "shrink + expand",
                   "tokens": T, "prefill_tokens": pre["T"] if pre else 0, "adapters": cfg["N"],
                   "adapters_touched": int(len(uniq)), "group": group,
                   "hip_graph": not args.no_graph, "timed_region_ms": t["timed_ms"], "wall_s_timed_region": t["wall_s"],
                   # the decode half alone: the layers' BGMV calls without gather, plan and prefill launches
                   "decode_only_token_projections_per_s": T * len(projs) * L / (tk["ms"] * 1e-3),
                   "decode_only_ms_per_step": tk["ms"]},
        "roofline": dict({"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "traffic_source": src, "kernel": kernel}, **extra),
        "cpu_baseline": None,
    }
    if args.eager and not args.no_graph:
        te = timed(step, max(5, min(reps, 50)), 2)
        out["config"]["eager_ms_per_step"] = te["ms"]
    return out


# ---------------------------------------------------------------------------------------------- cold start
def bench_coldstart(args, dev, steps, warmup):
    """The reference's one published claim, on its own shape (config/ali-a10.yml: hidden 4096, one request of 64
    tokens, 8 tokens per host worker; rank 64, 32 layers, q/k/v): the latency of a prefill whose adapter is
    (a) cached in the pool, (b) loading while the prefill runs, the layers whose rows have not landed served by the
    host workers (CPU-assisted), (c) loaded first, then prefilled (on demand), and (d) loaded layer 0 first with
    every layer waiting on the device for its own rows (pipelined; no counterpart in the reference).  README.md:86-89
    expects cached < CPU-assisted < on-demand.  One request = admit, then per layer: path choice, base q/k/v projections
    (torch.mm), LoRA delta added (SGMV or collected from the host workers).  The rest of a transformer layer is not
    part of the loop, so the load has less to hide behind here than in a serving stack."""
    import statistics

    import torch

    import mlora
    L, H, r, tkn, cap = 32, 4096, 64, 64, 8
    names = ("q", "k", "v")
    pool = mlora.AdapterPool(L, {p: (H, H) for p in names}, n_slots=2, n_pages=2 * (r // 8), page_rows=8, max_rank=r,
                             dtype=torch.float16, device=dev)
    cfg = dict(batch_size=1, lora_num=8, tp_degree=1, hidden_dim=H, lora_rank=r, token_per_lora=cap, n_layers=L)
    cpu = mlora.Lora_CPU(cfg, gpu_id=0, device=dev)
    cs = mlora.ColdStartPrefill(pool, cpu, max_adapters=1)
    gen = torch.Generator().manual_seed(6006)
    w = {p: (torch.randn(L, H, r, generator=gen) * 0.001, torch.randn(L, r, H, generator=gen) * 0.001) for p in names}
    cs.register_adapter(0, w, 1.0)
    n_threads = max(1, min(host_cores()["usable_by_this_process"], 64))
    cs.start_workers(n_threads)
    dgen = torch.Generator(device=dev)
    dgen.manual_seed(6007)
    W = [[(torch.randn(H, H, device=dev, generator=dgen) / H ** 0.5).half() for _ in names] for _ in range(L)]
    xs = [torch.randn(tkn, H, device=dev, generator=dgen).half() for _ in range(L)]
    qkv = [torch.empty(tkn, H, device=dev, dtype=torch.float16) for _ in names]

    def request(mode):
        if mode != "cached":
            cs.evict(0)
        torch.cuda.synchronize()
        c0 = cs.count_use_cpu_lora
        t0 = time.perf_counter()
        cs.admit([0], tkn, mode)
        for l in range(L):
            path = cs.start_layer(xs[l], l)
            for i in range(3):
                torch.mm(xs[l], W[l][i], out=qkv[i])
            cs.finish_layer(path, xs[l], l, qkv)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3, cs.count_use_cpu_lora - c0

    try:
        reps = max(steps, 20)
        res = {}
        request("on_demand")                                   # the adapter is resident from here on
        for mode in ("cached", "cpu_assisted", "on_demand", "pipelined"):
            for _ in range(max(warmup, 3)):
                request(mode)
            runs = [request(mode) for _ in range(reps)]
            ms = sorted(t for t, _ in runs)
            res[mode] = {"ms": statistics.median(ms), "p10": ms[len(ms) // 10], "p90": ms[(9 * len(ms)) // 10],
                         "layers_on_host_workers": sum(c for _, c in runs) / len(runs)}
    finally:
        cs.stop_workers()
        cpu.close()
    nbytes = cs.host[0].nbytes
    load_ms = max(res["on_demand"]["ms"] - res["cached"]["ms"], 1e-6)
    gbs = nbytes / (load_ms * 1e-3) / 1e9
    holds = res["cached"]["ms"] < res["cpu_assisted"]["ms"] < res["on_demand"]["ms"]
    return {"metric": "prefill latency of a request whose adapter is cold (CPU-assisted path)", "value": res["cpu_assisted"]["ms"],
            "unit": "ms", "n_gpus": 1, "steps": reps, "warmup": max(warmup, 3), "ms_per_step": res["cpu_assisted"]["ms"],
            "ms_per_step_spread": {k: res["cpu_assisted"][k] for k in ("p10", "p90")}, "higher_is_better": False,
            "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": "cold start: one request of 64 tokens, hidden 4096, rank-64 adapter for q/k/v of 32 layers "
                                   f"({nbytes / 1e6:.1f} MB), 8 tokens per host worker, {n_threads} worker threads; per layer: base q/k/v "
                                   "projections + LoRA delta", "form": "cached | CPU-assisted | on demand | pipelined (layer 0 first, each layer waits for its own rows on the device)",
                       "cached_ms": res["cached"]["ms"], "cpu_assisted_ms": res["cpu_assisted"]["ms"],
                       "on_demand_ms": res["on_demand"]["ms"], "pipelined_ms": res["pipelined"]["ms"], "ordering_holds": holds,
                       "expected_ordering": "cached < CPU-assisted < on-demand (README.md:86-89 of the reference)",
                       "layers_on_host_workers_cpu_assisted": res["cpu_assisted"]["layers_on_host_workers"],
                       "spread": {m: {k: res[m][k] for k in ("p10", "p90")} for m in res}, "worker_threads": n_threads},
            "roofline": {"bound": "pcie", "achieved": gbs, "peak": 64.0, "unit": "GB/s", "frac": gbs / 64.0, "traffic": None,
                         "traffic_source": None, "kernel": "adapter load behind the on-demand request: (on-demand - cached) latency"},
            "cpu_baseline": None}


# ---------------------------------------------------------------------------------------------- arrival trace
def bench_trace(args, dev, steps, warmup, n_adapters=128, n_slots=64):
    """bench.py leg `maf_trace`: the decode steps of the reference's 512-arrival-rate trace (adapter ids from its
    popularity vector of `n_adapters` adapters) on Llama-7B q/k/v shapes, rank 16, a pool of `n_slots` slots, eager
    launches (the batch changes every step); reports decode steps per second and the per-layer call time."""
    import numpy as np
    import torch

    from mlora import workloads
    from mlora.trace_driver import TraceRunner, draw_output_lengths, simulate
    root = os.path.join(ROOT, "tests", "golden")
    times = np.load(os.path.join(root, "maf_trace_512.npy"), allow_pickle=False)
    pop = np.load(os.path.join(root, f"maf_popularity_{n_adapters}.npy"), allow_pickle=False)
    ids = workloads.draw_lora_ids(pop, len(times), seed=0)
    lens = draw_output_lengths(len(times), mean=256.0, seed=1)
    sim = simulate(times, ids, lens, step_s=0.03, running_max_req_size=256, max_prefill_batch_size=8)
    decode = [s for s in sim if s.kind == "decode" and len(s.lora_ids) > 0]
    L, H, r = 32, 4096, 16
    run = TraceRunner(L, H, r, n_slots, device=dev, max_batch=256)
    n_steps = min(len(decode), max(steps, 200))
    first = min(len(decode) - n_steps, 400)                  # past the ramp-up of the trace
    window = decode[first:first + n_steps]
    warm = decode[max(0, first - max(warmup, 20)):first]
    # the adapters live in pinned host memory before the replay starts (drawing their weights is not part of a step)
    for a in sorted({int(a) for s in warm + window for a in s.lora_ids}):
        run.host[a] = run.loader.stage(run.adapter_weights(a), run.rank, run.scaling)
    for s in warm:
        run.decode_step(s.lora_ids)
    torch.cuda.synchronize()
    loads0 = run.residency.loads
    per = []
    t0 = time.perf_counter()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for s in window:
        t1 = time.perf_counter()
        run.decode_step(s.lora_ids)
        per.append((time.perf_counter() - t1) * 1e3)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    gpu_ms = e0.elapsed_time(e1)
    sizes = np.array([len(s.lora_ids) for s in window])
    touched = np.array([len(set(s.lora_ids.tolist())) for s in window])
    tokproj = int(sizes.sum()) * 3 * L
    s_per = sorted(per)
    pick = lambda q: s_per[min(len(s_per) - 1, int(round(q * (len(s_per) - 1))))]
    ms_per_step = wall * 1e3 / n_steps
    # algorithmic bytes of the window: per step and layer, x once per projection, y read + written, touched adapters' rows once
    alg = float(sum(3 * (t * H * 2 + 2 * t * H * 2 + u * r * 2 * H * 2 + 4 * t) for t, u in zip(sizes, touched))) * L
    achieved = alg / (gpu_ms * 1e-3) / 1e9
    return {"metric": "decode steps per second on the reference's arrival trace", "value": n_steps / wall, "unit": "steps/s",
            "n_gpus": 1, "steps": n_steps, "warmup": warmup, "ms_per_step": ms_per_step,
            "ms_per_step_spread": {"p10": pick(0.1), "p50": pick(0.5), "p90": pick(0.9)}, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": f"maf_trace_512 arrivals, adapter per request from popularity_{n_adapters}, continuous batching "
                                   f"(256 running, 8 admitted per step), Llama-7B q/k/v 4096->4096, rank 16, {n_slots}-slot paged pool, "
                                   "32 layers, eager launches", "form": "gather + one BGMV call per layer, swap-in on miss",
                       "steps_in_trace": len(decode), "tokens": float(sizes.mean()), "adapters_touched_per_step": float(touched.mean()),
                       "swap_ins": run.residency.loads - loads0, "token_projections_per_s": tokproj / wall,
                       "gpu_ms_per_step": gpu_ms / n_steps},
            "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                         "traffic": None, "traffic_source": None,
                         "kernel": "gather + 32 x BGMV call (q, k, v), batch changing every step, eager",
                         "algorithmic_bytes_per_step": alg / n_steps},
            "cpu_baseline": None}


def leg_of(line):
    """The part of a workload's line that goes into the headline's `legs` object."""
    keep = {k: line[k] for k in ("metric", "value", "unit", "ms_per_step", "ms_per_step_spread", "steps", "dtype")}
    keep["workload"] = line["config"]["workload"]
    keep["form"] = line["config"].get("form")
    for k in ("cached_ms", "cpu_assisted_ms", "on_demand_ms", "pipelined_ms", "ordering_holds", "layers_on_host_workers_cpu_assisted", "eager_ms_per_step", "paged_call_same_batch_ms_per_step", "ratio_to_paged_call", "library_gemm_then_sgmv_ms", "speedup_over_library_gemm_then_sgmv", "tokens", "adapters_touched",
              "steps_in_trace", "adapters_touched_per_step", "swap_ins"):
        if k in line["config"]:
            keep[k] = line["config"][k]
    keep["roofline"] = line["roofline"]
    return keep


SINGLE = ["c1", "c2", "c3", "c4", "c5", "maf128", "maf256", "maf512", "maf_trace", "swap", "assist", "f1", "reflayout", "coldstart"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--layers", type=int, default=0, help="layers per step (0 = the workload's own count)")
    ap.add_argument("--group", type=int, default=-1,
                    help="tokens of one adapter per work item (0 = no plan, one token each; default: by batch size)")
    ap.add_argument("--split", action="store_true", help="decode: force the shrink + expand pair also where the host layer would pick the fused launch")
    ap.add_argument("--fused", action="store_true", help="decode: one fused launch per layer instead of the shrink + expand pair; c4: one SGMV call per projection "
                         "instead of one call over the seven")
    ap.add_argument("--one-stream", action="store_true", help="c5: decode and prefill launches of a layer one after the other on one stream "
                                                              "instead of side by side on two")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--eager", action="store_true", help="decode: also time the step launched eagerly (config.eager_ms_per_step)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-legs", action="store_true", help="default run: the config-5 headline alone")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run three plain 256 MiB device copies (known size) so that a counter run can be scaled")
    ap.add_argument("--workload", default="all", choices=["all"] + SINGLE,
                    help="all (default) = config 5 as the headline plus the legs c1, c2, c3, c4, f1, reflayout, maf_trace, coldstart; a name = that "
                         "workload alone: c1..c3, c5 decode BGMV; c4 prefill SGMV on Llama-13B shapes; mafN = decode batch drawn from the "
                         "reference's adapter-popularity vector of N adapters; maf_trace = continuous-batching decode sequence from the "
                         "reference's arrival trace; swap = adapter swap-in from pinned host memory; assist = CPU-assist transport; "
                         "f1 = base projection + LoRA in one pass on the config-4 batch; reflayout = the reference's pool layout and call; "
                         "coldstart = prefill latency with the adapter cached, loading (CPU-assisted) and loaded on demand")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch

    import mlora

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    mlora._ext.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.calib_copy:
        src = torch.ones(128 << 20, dtype=torch.float16, device=dev)      # 256 MiB read + 256 MiB written per copy
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    def one(workload, steps, warmup, min_ms, cpu):
        if workload == "c4":
            return bench_c4(args, dev, steps, warmup, min_ms, cpu)
        if workload == "f1":
            return bench_f1(args, dev, steps, warmup, min_ms, cpu)
        if workload == "reflayout":
            return bench_reflayout(args, dev, steps, warmup, min_ms)
        if workload == "maf_trace":
            return bench_trace(args, dev, steps, warmup)
        if workload == "coldstart":
            return bench_coldstart(args, dev, steps, warmup)
        if workload == "swap":
            return bench_swap(args, dev)
        if workload == "assist":
            return bench_assist(args, dev)
        line = bench_decode(args, dev, workload, steps, warmup, min_ms)
        if cpu:
            log("timing the CPU baseline ...")
            line["cpu_baseline"] = cpu_baseline()
        return line

    if args.workload != "all":
        print(json.dumps(one(args.workload, args.steps, args.warmup, 0.0, not args.no_cpu)), flush=True)
        return

    t_start = time.perf_counter()
    legs = {}
    ceiling = stream_ceiling(dev)
    if not args.no_legs:
        args.eager = True
        for w in ("c1", "c2", "c3", "c4", "f1", "reflayout", "maf_trace", "coldstart"):
            log(f"leg {w} ...")
            try:
                legs[w] = leg_of(one(w, args.steps, args.warmup, MIN_LEG_MS, False))
            except ImportError as exc:                    # a leg whose driver is not in this tree is reported, not hidden
                legs[w] = {"error": str(exc)}
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
        args.eager = False
    log("headline: config 5 ...")
    line = bench_decode(args, dev, "c5", args.steps, args.warmup, 0.0)
    line["stream_ceiling"] = ceiling
    if not args.no_cpu:
        log("timing the CPU baseline ...")
        line["cpu_baseline"] = cpu_baseline()
    # The legs' figures as flat scalars of `config` (nested objects may be dropped by whoever stores the line):
    # fraction of the HBM peak for every leg that is bound by it, MFMA figures for the prefill legs.
    flat = line["config"]
    flat["c5_decode_hbm_frac"] = line["roofline"]["frac"]
    flat["c5_decode_launch_us"] = line["roofline"]["launch_us"]
    flat["c5_whole_step_hbm_frac"] = line["roofline"]["whole_step"]["frac"]
    for w, leg in legs.items():
        if "error" in leg:
            flat[f"{w}_error"] = leg["error"]
            continue
        rf = leg["roofline"]
        flat[f"{w}_ms_per_step"] = leg["ms_per_step"]
        if rf["bound"] == "hbm":
            flat[f"{w}_hbm_frac"] = rf["frac"]
        if w == "c1":
            # 2.9 MB per call = 0.36 us at the HBM peak: a single launch cannot be that short, whatever the kernel
            flat["c1_note"] = "latency-scale op: bounded by one kernel launch, not by HBM"
        if "launch_us" in rf:
            flat[f"{w}_launch_us"] = rf["launch_us"]
        if w == "c4":
            flat["c4_tflops"] = rf["mfma_tflops"]
            flat["c4_mfma_frac"] = rf["mfma_frac"]
            flat["c4_mfma_ceiling"] = rf["mfma_frac_ceiling"]
        if w == "f1":
            flat["f1_tflops"] = rf["achieved"]
            flat["f1_mfma_frac"] = rf["frac"]
        if w == "coldstart":
            for k in ("cached_ms", "cpu_assisted_ms", "on_demand_ms", "pipelined_ms", "ordering_holds"):
                flat[f"coldstart_{k}"] = leg.get(k)
    flat["bench_wall_s"] = time.perf_counter() - t_start
    # key order of the printed line: the legs first, the headline's own fields after them, `config` (with the flat scalars) last
    ordered = {"legs": legs}
    ordered.update({k: v for k, v in line.items() if k != "config"})
    ordered["config"] = line["config"]
    print(json.dumps(ordered), flush=True)


if __name__ == "__main__":
    main()
