#!/usr/bin/env python3
"""Benchmark of the multi-LoRA decode hot path on one MI355X.

Workload (the configuration the metric is quoted on): decode BGMV over the Llama-7B attention
projections q/k/v/o (4096 -> 4096 each), 256 decode tokens, 64 rank-16 fp16 adapters in one paged
pool, adapter per token ~ Zipf(1.0), scaling 2.0.  One step = one decode step's LoRA work: the
adapter-pool gather once, then for each of the 32 layers one BGMV call (a shrink launch and an
expand launch, or one fused launch with --fused) covering that layer's q, k, v (shared input) and
o (own input), accumulating into the base projection outputs.
Every layer has its own pool slabs, inputs and outputs (about 2.4 GB in all), so a step streams
from HBM rather than from the 256 MB last-level cache.

Prints one JSON line: throughput in token-projections/s, the HBM roofline of the BGMV call
(algorithmic bytes / measured duration of one layer's launches) and the CPU baseline (the CPU-assisted path's
arithmetic timed on the host cores).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "ae-296_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_BF16_TFLOPS = 2500.0      # dense bf16 / fp16 MFMA peak of the device
# HBM bytes per BGMV call (shrink + expand launch) of the default workload, from the two counter runs summarised in
# profiles/bgmv_c2_bench.txt (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, factors from a 256 MiB copy in the
# same runs).  Reported as roofline.traffic only when the run is that same configuration.
MEASURED_TRAFFIC_C2 = 81.78e6
MEASURED_TRAFFIC_C4_STEP = 2906.7e6


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def algorithmic_bytes(T, projs, ranks_of_unique, elt=2):
    """Per projection call: x read + y read and write + every touched adapter's rows once + indices."""
    total = 0
    for hin, hout in projs:
        total += T * hin * elt + 2 * T * hout * elt + int(sum(ranks_of_unique)) * (hin + hout) * elt + 4 * T
    return total


def cpu_baseline(seconds=12.0):
    """The reference's CPU-assisted LoRA arithmetic (x.float() @ down @ up -> half, one task per
    request chunk) on config 1: 32 tokens, 8 rank-16 adapters, 4096 -> 4096, timed on the host cores."""
    import numpy as np
    from oracle import oracle as orc
    rng = np.random.default_rng(1001)
    T, N, r, H = 32, 8, 16, 4096
    down = (rng.standard_normal((N, H, r)) * 0.02).astype(np.float32)
    up = (rng.standard_normal((N, r, H)) * 0.02).astype(np.float32)
    x = rng.standard_normal((T, H)).astype(np.float16).view(np.uint16)
    req_adapter = rng.integers(0, N, T).astype(np.int32)
    cores = max(1, min(16, os.cpu_count() or 1))
    pool = orc.CpuLoraPool(cores)                                       # persistent workers, as the reference's are
    out_buf = np.empty((T, H), np.uint16)
    pool.run(x, down, up, req_adapter, 1, 8, out_buf)                  # warm-up
    n, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        pool.run(x, down, up, req_adapter, 1, 8, out_buf)
        n += 1
    dt = time.perf_counter() - t0
    pool.close()
    out = {"value": T * n / dt, "unit": "token-projections/s", "cores": cores, "kind": "port",
           "sample": f"config 1 (32 decode tokens, 8 rank-16 adapters, 4096->4096, fp32 weights), {n} repetitions "
                     f"in {dt:.1f} s, one task per token over {cores} persistent worker threads"}
    # The same expression through the library the reference's workers call (torch CPU matmul, one thread per
    # worker as shared_tensor.py:35 / runServerCPULoRA.py:83 pin it): one request per call, a few seconds.
    import torch
    prev = torch.get_num_threads()
    try:
        torch.set_num_threads(1)
        xt = torch.from_numpy(x.view(np.float16).copy())
        dn, upt = torch.from_numpy(down), torch.from_numpy(up)
        m, t1 = 0, time.perf_counter()
        while time.perf_counter() - t1 < 3.0:
            for t in range(T):
                a = int(req_adapter[t])
                (xt[t:t + 1].float() @ dn[a] @ upt[a]).half()
            m += 1
        d1 = time.perf_counter() - t1
        out["torch_cpu_one_thread"] = {"value": T * m / d1, "unit": "token-projections/s", "cores": 1,
                                       "sample": f"x.float() @ down @ up -> half per request with torch on one thread, "
                                                 f"{m} repetitions in {d1:.1f} s"}
    finally:
        torch.set_num_threads(prev)
    return out


def cpu_baseline_prefill(with_base, seconds=10.0):
    """The oracle (scalar C, one core) on a bounded sample of the config-4 prefill: one segment (128 tokens, or
    32 with the base product) on one rank-64 adapter, q projection 5120 -> 5120, bf16 -- the LoRA delta added
    into y (`with_base` False, the SGMV step) or y = x W + delta (`with_base` True).  Reported in the GPU
    line's unit (TFLOP/s)."""
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


def bench_c4(args, dev):
    """Prefill SGMV, config 4: Llama-13B shapes (hidden 5120, MLP 13824), 16 requests with prompt lengths
    U[128, 1024], each bound to one of 32 rank-64 adapters, bf16, tokens packed per request.  One step =
    the seven projections of one layer (q, k, v, o, gate, up, down), each one mlora_sgmv call."""
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
    ss, sl, sa = (torch.from_numpy(a).to(dev) for a in (starts, lens, adapters))
    gen = torch.Generator(device=dev)
    gen.manual_seed(4004)
    x = {h: torch.randn(T, h, device=dev, generator=gen).bfloat16() for h in (5120, 13824)}
    y = {p: torch.randn(T, projections[p][1], device=dev, generator=gen).bfloat16() for p in projections}
    # q, k, v read the attention input, gate and up the MLP input; o and down have inputs of their own
    x_o = torch.randn(T, 5120, device=dev, generator=gen).bfloat16()
    x_ffn = torch.randn(T, 5120, device=dev, generator=gen).bfloat16()
    x_in = {"q": x[5120], "k": x[5120], "v": x[5120], "o": x_o, "gate": x_ffn, "up": x_ffn, "down": x[13824]}
    ws = mlora.sgmv_workspace(T, 16, dev, n_proj=len(projections))
    names = list(projections)

    def step():
        plan = mlora.plan_prefill(ss, sl, sa, T, pool, workspace=ws)      # once per batch, shared by the projections
        if args.fused:                                                     # one call per projection (3 launches each)
            for p, (hin, hout) in projections.items():
                mlora.sgmv(y[p], x[hin], pool, 0, p, accumulate=True, plan=plan)
        else:                                                              # all seven in one call (3 launches)
            mlora.sgmv_multi([y[p] for p in names], [x_in[p] for p in names], pool, 0, names, plan)

    step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    ms_per_step = e0.elapsed_time(e1) / args.steps
    flops = sum(2.0 * 64 * (hin + hout) * T for hin, hout in projections.values())
    uniq = np.unique(adapters)
    alg = sum(T * hin * 2 + 2 * T * hout * 2 + len(uniq) * 64 * (hin + hout) * 2 + 4 * T + 12 * 16
              for hin, hout in projections.values())
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    gbs = alg / (ms_per_step * 1e-3) / 1e9
    out = {"metric": "SGMV prefill throughput", "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"workload": "config 4: prefill SGMV, Llama-13B q/k/v/o/gate/up/down, 16 requests U[128,1024], "
                                  "32 rank-64 adapters, bf16", "tokens": T, "segments": 16},
           "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                        "traffic": None if args.fused else MEASURED_TRAFFIC_C4_STEP, "kernel": "sgmv plan (once) + 7 x (shrink, reduce, expand)" if args.fused else
                                  "sgmv plan (once) + one shrink, reduce and expand launch over the 7 projections",
                        "algorithmic_bytes_per_step": alg, "mfma_tflops": tflops, "mfma_frac_of_2500": tflops / 2500.0},
           "cpu_baseline": None if args.no_cpu else cpu_baseline_prefill(False)}
    print(json.dumps(out), flush=True)


def bench_f1(args, dev):
    """Base projection + LoRA in one pass on the config-4 batch (Llama-13B shapes, 16 requests U[128, 1024],
    32 rank-64 adapters, bf16): one step = q, k, v, o, gate, up, down of one layer, y = x W + delta, as one
    mlora_gemm_lora_planned call (shrink, scaled reduce, one GEMM launch).  The same step as the reference runs
    it -- library GEMM per projection, then the SGMV kernels adding the delta -- is timed beside it."""
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
    ss, sl, sa = (torch.from_numpy(a).to(dev) for a in (starts, lens, adapters))
    gen = torch.Generator(device=dev)
    gen.manual_seed(4004)
    x = {h: torch.randn(T, h, device=dev, generator=gen).bfloat16() for h in (5120, 13824)}
    x_o = torch.randn(T, 5120, device=dev, generator=gen).bfloat16()
    x_ffn = torch.randn(T, 5120, device=dev, generator=gen).bfloat16()
    x_in = {"q": x[5120], "k": x[5120], "v": x[5120], "o": x_o, "gate": x_ffn, "up": x_ffn, "down": x[13824]}
    names = list(projections)
    w = {p: (torch.randn(projections[p], device=dev, generator=gen) / projections[p][0] ** 0.5).bfloat16() for p in names}
    y = {p: torch.empty(T, projections[p][1], device=dev, dtype=torch.bfloat16) for p in names}
    ws = mlora.sgmv_workspace(T, 16, dev, n_proj=len(names))

    def fused():
        plan = mlora.plan_prefill(ss, sl, sa, T, pool, workspace=ws, aligned=True)
        mlora.gemm_lora([y[p] for p in names], [x_in[p] for p in names], [w[p] for p in names], pool, 0, names, plan)

    def unfused():
        plan = mlora.plan_prefill(ss, sl, sa, T, pool, workspace=ws)
        for p in names:
            torch.mm(x_in[p], w[p], out=y[p])
        mlora.sgmv_multi([y[p] for p in names], [x_in[p] for p in names], pool, 0, names, plan)

    def base_only():
        for p in names:
            torch.mm(x_in[p], w[p], out=y[p])

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    ms_unfused = timed(unfused)
    ms_base = timed(base_only)
    ms_per_step = timed(fused)
    flops = sum(2.0 * T * hin * hout + 2.0 * 64 * (hin + hout) * T for hin, hout in projections.values())
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    out = {"metric": "base projection + LoRA prefill throughput", "value": tflops, "unit": "TFLOP/s", "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"workload": "config-4 batch with base weights: Llama-13B q/k/v/o/gate/up/down, 16 requests U[128,1024], "
                                  "32 rank-64 adapters, bf16; y = x W + delta in one pass", "tokens": T, "segments": 16,
                      "library_gemm_then_sgmv_ms": ms_unfused, "library_gemm_alone_ms": ms_base,
                      "speedup_over_library_gemm_then_sgmv": ms_unfused / ms_per_step},
           "roofline": {"bound": "mfma", "achieved": tflops, "peak": MFMA_PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                        "frac": tflops / MFMA_PEAK_BF16_TFLOPS, "traffic": None,
                        "kernel": "sgmv shrink + scaled reduce + gemm_lora_kernel (one launch over the 7 projections)",
                        "flops_per_step": flops},
           "cpu_baseline": None if args.no_cpu else cpu_baseline_prefill(True)}
    print(json.dumps(out), flush=True)


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
    out = {"metric": "adapter swap-in throughput (host pinned -> pool pages)", "value": gbs, "unit": "GB/s", "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup, "ms_per_step": total * 1e3, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "u16", "data": "synthetic",
           "config": {"workload": "swap-in of one rank-64 adapter, q/k/v, 32 layers, hidden 4096, fp16",
                      "bytes_per_adapter": nbytes, "layers_per_copy": loader.layers_per_copy,
                      "ms_until_layers_8_15_ready": first * 1e3, "ms_host_time_to_issue": issue * 1e3},
           "roofline": {"bound": "pcie", "achieved": gbs, "peak": 64.0, "unit": "GB/s", "frac": gbs / 64.0, "traffic": None,
                        "kernel": "host->device copies (copy engine) + scatter_kernel"},
           "cpu_baseline": {"value": nbytes / ref_t / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                            "sample": f"the swapper's copy pattern (pageable host tensors, one copy and one slice assignment per "
                                      f"layer and tensor) restated with torch, {n_ref} adapters, {ref_t * 1e3:.2f} ms each"}}
    print(json.dumps(out), flush=True)


def bench_assist(args, dev):
    """CPU-assist transport alone (no worker arithmetic): hidden states of a prefill batch to the host request
    slots plus the wake-up codes, and the q/k/v result slots back to the device.  Shape of the reference's
    CPU-assisted prefill: hidden 4096, slots of 256 tokens, 64 tokens per worker; 8 requests of 256 tokens.
    Beside it, the reference's call pattern restated with torch (one device->host copy per request, one
    host->device copy per finished chunk and projection, lora_cpu.py:176-232)."""
    import torch

    import mlora
    B, tkn, H, cap = 8, 256, 4096, 64
    cfg = dict(batch_size=B, lora_num=64, tp_degree=1, hidden_dim=H, lora_rank=16, token_per_lora=cap, n_layers=32)
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
    out = {"metric": "CPU-assist transport throughput (device <-> pinned host slots)", "value": gbs, "unit": "GB/s", "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup, "ms_per_step": t_exp + t_imp, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "u16", "data": "synthetic",
           "config": {"workload": "8 requests x 256 tokens, hidden 4096: export 16.8 MB + wake-up codes, import q/k/v 50.3 MB",
                      "export_ms": t_exp, "import_ms": t_imp, "export_GBs": b_exp / t_exp / 1e6, "import_GBs": b_imp / t_imp / 1e6},
           "roofline": {"bound": "pcie", "achieved": gbs, "peak": 64.0, "unit": "GB/s", "frac": gbs / 64.0, "traffic": None,
                        "kernel": "assist_export_kernel + assist_signal_kernel, assist_import_kernel"},
           "cpu_baseline": {"value": (b_exp + b_imp) / ((r_exp + r_imp) * 1e-3) / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                            "sample": f"the reference's call pattern restated with torch: {B} copies out ({r_exp:.3f} ms), "
                                      f"{3 * B * cpr} synchronous chunk copies back ({r_imp:.3f} ms)"}}
    print(json.dumps(out), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--layers", type=int, default=0, help="layers per step (0 = the workload's own count)")
    ap.add_argument("--group", type=int, default=-1,
                    help="tokens of one adapter per work item (0 = no plan, one token each; default: by batch size)")
    ap.add_argument("--split", action="store_true", help="decode: force the shrink + expand pair also where the host layer would pick the fused launch")
    ap.add_argument("--fused", action="store_true", help="decode: one fused launch per layer instead of the shrink + expand pair; c4: one SGMV call per projection "
                         "instead of one call over the seven")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run three plain 256 MiB device copies (known size) so that a counter run can be scaled")
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c3", "c4", "c5", "maf128", "maf256", "maf512", "swap", "assist", "f1"],
                    help="c2 = decode BGMV (the headline metric); c1, c3 = the other decode configurations; "
                         "c4 = prefill SGMV on Llama-13B shapes; c5 = full 32-layer step with 1000 adapters (about 165 GB); "
                         "mafN = decode batch drawn from the reference's adapter-popularity vector of N adapters; "
                         "swap = adapter swap-in from pinned host memory; assist = CPU-assist transport; "
                         "f1 = base projection + LoRA in one pass on the config-4 batch, with the library GEMM + SGMV sequence timed beside it")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import mlora
    from mlora import workloads

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
    if args.workload == "c4":
        return bench_c4(args, dev)
    if args.workload == "f1":
        return bench_f1(args, dev)
    if args.workload == "swap":
        return bench_swap(args, dev)
    if args.workload == "assist":
        return bench_assist(args, dev)
    return bench_decode(args, dev)


# Decode workloads.  `inputs` names the activation tensor each projection reads (projections that
# read the same tensor in the model share it here).  `layers` is chosen so that a step's working
# set is far larger than the 256 MB last-level cache.
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


def bench_decode(args, dev):
    import numpy as np
    import torch

    import mlora
    from mlora import workloads

    cfg = DECODE[args.workload]
    if args.group < 0:
        args.group = mlora.ops.default_group(cfg["T"])
    L = args.layers if args.layers > 0 else cfg["layers"]
    shapes = workloads.LLAMA7B_ATTN if cfg["shapes"] == "7b_attn" else workloads.LLAMA7B_ALL
    projs = cfg["projs"]
    shapes = {p: shapes[p] for p in projs}
    rng = np.random.default_rng(cfg["seed"])
    ranks = cfg["ranks"] if cfg["ranks"] is not None else rng.choice([8, 16, 32, 64], size=cfg["N"]).astype(np.int32)
    log(f"building {args.workload} with {L} layers ...")
    lora_ids = None
    if cfg.get("popularity"):
        lora_ids = workloads.draw_lora_ids(np.load(cfg["popularity"], allow_pickle=False), cfg["T"], seed=0)
    wl = workloads.make_decode(args.workload, shapes, L, cfg["T"], cfg["N"], ranks, cfg["alpha"], seed=cfg["seed"],
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
    plan = mlora.plan_decode(tok, pool, group=args.group) if args.group else None
    fused = bool(args.fused or plan is None or
                 (not args.split and mlora.ops.decode_fused(T, args.group, len(projs), pool.n_slots)))

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

    def bgmv_layers():
        for l in range(L):
            mlora.bgmv(ys[l], [xs[l][_IN[p]] for p in projs], pool, l, projs, tok, plan=plan, fused=fused)

    def step():
        if plan is not None:
            mlora.plan_decode(tok, pool, group=args.group, out=plan)
        if pre is None:
            bgmv_layers()
            return
        pplan = mlora.plan_prefill(pre["ss"], pre["sl"], pre["sa"], pre["T"], pool, workspace=pre["ws"])
        for l in range(L):
            mlora.bgmv(ys[l], [xs[l][_IN[p]] for p in projs], pool, l, projs, tok, plan=plan, fused=fused)
            mlora.sgmv_multi([pre["y"][p] for p in projs], [pre["x"][_IN[p]] for p in projs], pool, l, projs, pplan)

    step()
    torch.cuda.synchronize()

    def make_runner(fn):
        if args.no_graph:
            return fn
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        return g.replay

    def timed(run, reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            run()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1)          # ms, on the stream the kernels run on

    run_step = make_runner(step)
    for _ in range(args.warmup):
        run_step()
    torch.cuda.synchronize()
    t_wall = time.perf_counter()
    ms = timed(run_step, args.steps)
    wall = time.perf_counter() - t_wall
    ms_per_step = ms / args.steps
    n_tok = T + (pre["T"] if pre else 0)
    value = n_tok * len(projs) * L / (ms_per_step * 1e-3)

    uniq = np.unique(wl.tok_adapter[wl.tok_adapter >= 0])
    shp = [shapes[p] for p in projs]
    alg = algorithmic_bytes(T, shp, wl.ranks[uniq])
    per_token_gather = sum(T * h[0] * 2 + 2 * T * h[1] * 2 + int(wl.ranks[wl.tok_adapter].sum()) * (h[0] + h[1]) * 2 + 4 * T
                           for h in shp)
    if pre is None:
        # The BGMV calls alone: the same layers without the gather, for the roofline figure.
        run_bgmv = make_runner(bgmv_layers)
        for _ in range(args.warmup):
            run_bgmv()
        ms_k = timed(run_bgmv, args.steps)
        launch_us = ms_k * 1e3 / (args.steps * L)
        achieved = alg / (launch_us * 1e-6) / 1e9
        kernel = ("bgmv_kernel" if fused else "bgmv_shrink_kernel + bgmv_expand_kernel (one layer's pair)") + \
                 f", {len(projs)} projections per call"
        extra = {"launch_us": launch_us, "algorithmic_bytes_per_launch": alg,
                 "per_token_gather_bytes_per_launch": per_token_gather}
    else:
        # Mixed step: decode and prefill bytes of all layers over the whole step (gather and plan included).
        pu = np.unique(pre["adapters"])
        alg_pre = algorithmic_bytes(pre["T"], shp, wl.ranks[pu]) + 12 * len(pre["adapters"]) * len(projs)
        alg_step = (alg + alg_pre) * L
        achieved = alg_step / (ms_per_step * 1e-3) / 1e9
        kernel = "whole step: gather + prefill plan + 32 x (decode pair + SGMV shrink, reduce, expand over 7 projections)"
        extra = {"algorithmic_bytes_per_step": alg_step, "decode_bytes_per_layer": alg, "prefill_bytes_per_layer": alg_pre}
    traffic = MEASURED_TRAFFIC_C2 if (args.workload == "c2" and args.group == 4 and L == 32 and not fused) else None

    out = {
        "metric": "BGMV decode throughput (LoRA-applied token-projections per second)",
        "value": value, "unit": "token-projections/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": cfg["desc"], "layers": L, "projections_per_call": len(projs),
                   "launches_per_step": L * (1 if fused else 2) + (1 if plan else 0) + ((1 + 3 * L) if pre else 0),
                   "form": "fused" if fused else "shrink + expand",
                   "tokens": T, "prefill_tokens": pre["T"] if pre else 0, "adapters": cfg["N"],
                   "adapters_touched": int(len(uniq)), "group": args.group,
                   "hip_graph": not args.no_graph, "wall_s_timed_region": wall},
        "roofline": dict({"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "kernel": kernel}, **extra),
        "cpu_baseline": None,
    }
    if not args.no_cpu:
        log("timing the CPU baseline ...")
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
