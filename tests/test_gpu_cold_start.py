"""Prefill during an adapter's cold start, composed: a 32-layer loop that asks per layer whether the adapter's rows have
landed (`use_gpu_pipeline`, lora_gpu.py:298-321) and serves q, k, v through the CPU-assisted path (host workers,
lora_cpu.py:138-276, app.py:102-143) or through the GPU path (SGMV on the pool pages), as
transformer_layer_infer.py:114-171 does.  Both paths must be taken while a load is in flight, every layer's q, k, v
must equal the oracle whichever path served it, and the two paths must agree with each other.

Expected values: CPU path -- the worker arithmetic (`orc.cpu_lora_worker`, fp32 weights, one rounding to fp16) added
to the base output in fp16, bit for bit; GPU path -- `orc.lora_apply_paged` (fp32 accumulation, one rounding) within
rtol 1e-2 / atol 1e-3.
"""
import numpy as np
import pytest
import torch

from gpu_common import ATOL, RTOL, say
from mlora import AdapterPool, ColdStartPrefill, Lora_CPU
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

L, H, R, CAP = 32, 512, 16, 8
NAMES = ("q", "k", "v")


def _bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def _setup(n_adapters, lora_num=16):
    pool = AdapterPool(L, {p: (H, H) for p in NAMES}, n_slots=4, n_pages=4 * R // 8 + 3, page_rows=8, max_rank=R,
                       dtype=torch.float16, device="cuda")
    cfg = dict(batch_size=4, lora_num=lora_num, tp_degree=1, hidden_dim=H, lora_rank=R, token_per_lora=CAP, n_layers=L)
    cpu = Lora_CPU(cfg)
    cs = ColdStartPrefill(pool, cpu, max_adapters=n_adapters)
    gen = torch.Generator().manual_seed(7)
    weights = []
    for aid in range(n_adapters):
        w = {p: ((torch.randn(L, H, R, generator=gen) * 0.05).half(), (torch.randn(L, R, H, generator=gen) * 0.05).half())
             for p in NAMES}
        cs.register_adapter(aid, w, scaling=2.0 if aid % 2 == 0 else 0.5)
        weights.append(w)
    cs.start_workers(4)
    return pool, cpu, cs, weights


def _expected(path, weights, adapter_ids, scalings, tkn, layer, proj, x_bits, y0_bits):
    """Bits (CPU path) or fp32 values (GPU path) of y0 + delta for the whole batch."""
    B = len(adapter_ids)
    if path == "cpu":
        out = np.empty_like(y0_bits)
        for b, aid in enumerate(adapter_ids):
            A, Bm = weights[aid][proj]
            down = A[layer].float().numpy()
            up = (Bm[layer].float() * scalings[aid]).numpy()
            for t0 in range(0, tkn, CAP):                          # one worker per chunk of <= CAP tokens
                sl = slice(b * tkn + t0, b * tkn + min(t0 + CAP, tkn))
                d = orc.cpu_lora_worker(np.ascontiguousarray(x_bits[sl]), down, up)
                out[sl] = (y0_bits[sl].view(np.float16) + d.view(np.float16)).view(np.uint16)    # q += q_lora, in fp16
        return out
    # GPU path: the oracle over a dense copy of the adapters of this batch
    a_rows = np.concatenate([_bits(weights[aid][proj][0][layer].t().contiguous()) for aid in adapter_ids])      # [r, H] rank rows
    b_rows = np.concatenate([_bits(weights[aid][proj][1][layer]) for aid in adapter_ids])
    tbl = np.arange(B * (R // 8), dtype=np.int32).reshape(B, R // 8)
    tok = np.repeat(np.arange(B, dtype=np.int32), tkn)
    want = orc.lora_apply_paged(x_bits, a_rows, b_rows, tok, tbl, tbl, np.full(B, R, np.int32),
                                np.array([scalings[a] for a in adapter_ids], np.float32), 8, orc.FP16, y0=y0_bits)
    return orc.from_bits(want, orc.FP16)


def test_cold_start_prefill_switches_paths_layer_by_layer():
    pool, cpu, cs, weights = _setup(2)
    scalings = {0: 2.0, 1: 0.5}
    adapter_ids, tkn = [1, 0], 24                                  # two requests, 24 tokens each: 3 chunks per request
    T = len(adapter_ids) * tkn
    gen = torch.Generator(device="cuda").manual_seed(3)
    xs = [torch.randn(T, H, device="cuda", generator=gen).half() for _ in range(L)]
    y0 = [[torch.randn(T, H, device="cuda", generator=gen).half() for _ in NAMES] for _ in range(L)]
    ys = [[y.clone() for y in layer] for layer in y0]
    # long copies ahead of the loads on the loader's stream (8 GB over the host link, well over 100 ms): the adapters'
    # rows cannot land before they are through, and the three layers below take a few milliseconds
    gate_host = torch.empty(1 << 30, dtype=torch.uint8, pin_memory=True)
    gate_dev = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    try:
        torch.cuda.synchronize()
        with torch.cuda.stream(cs.loader.stream):
            for _ in range(8):
                gate_dev.copy_(gate_host, non_blocking=True)
        say("cold start: admit with the loads in flight")
        cs.admit(adapter_ids, tkn, mode="cpu_assisted")
        paths = []
        for layer in range(L):
            if layer == 3:
                # from here on the loads are in (the host waits once): the remaining layers find their rows
                for t in cs.tickets:
                    t.wait()
            say(f"cold start: layer {layer}")
            path = cs.start_layer(xs[layer], layer)
            cs.finish_layer(path, xs[layer], layer, ys[layer])
            paths.append(path)
        torch.cuda.synchronize()
        assert paths[:3] == ["cpu"] * 3 and paths[3:] == ["gpu"] * (L - 3), paths
        assert cs.count_use_cpu_lora == 3 and cs.count_use_gpu_lora == L - 3
        for layer in range(L):
            x_bits = _bits(xs[layer])
            for q, p in enumerate(NAMES):
                want = _expected(paths[layer], weights, adapter_ids, scalings, tkn, layer, p, x_bits, _bits(y0[layer][q]))
                if paths[layer] == "cpu":
                    assert np.array_equal(_bits(ys[layer][q]), want), (layer, p)
                else:
                    got = ys[layer][q].float().cpu().numpy()
                    err = np.abs(got - want)
                    assert np.all(err <= ATOL + RTOL * np.abs(want)), (layer, p, float(err.max()))

        # the two paths on the same layer and input agree (two roundings against one)
        for layer in (0, 17, 31):
            a = [y.clone() for y in y0[layer]]
            b = [y.clone() for y in y0[layer]]
            say(f"cold start: both paths on layer {layer}")
            cs.finish_layer(cs.start_layer(xs[layer], layer, force="cpu"), xs[layer], layer, a)
            cs.finish_layer(cs.start_layer(xs[layer], layer, force="gpu"), xs[layer], layer, b)
            torch.cuda.synchronize()
            for ya, yb in zip(a, b):
                assert torch.allclose(ya.float(), yb.float(), rtol=RTOL, atol=ATOL)

        # a second batch on the now cached adapters takes the GPU path everywhere; an evicted one loads again
        cs.admit([0, 1], tkn, mode="cached")
        assert cs.use_gpu_pipeline(0) and cs.use_gpu_pipeline(L - 1)
        cs.evict(1)
        with pytest.raises(RuntimeError):
            cs.admit([0, 1], tkn, mode="cached")
        cs.admit([0, 1], tkn, mode="on_demand")
        ys2 = [y.clone() for y in y0[9]]
        cs.finish_layer(cs.start_layer(xs[9], 9), xs[9], 9, ys2)
        torch.cuda.synchronize()
        want = _expected("gpu", weights, [0, 1], scalings, tkn, 9, "k", _bits(xs[9]), _bits(y0[9][1]))
        err = np.abs(ys2[1].float().cpu().numpy() - want)
        assert np.all(err <= ATOL + RTOL * np.abs(want))
        # pipelined: layer 0 is loaded first and every layer's launch waits on the device for its own rows; no host worker
        cs.evict(0)
        cs.evict(1)
        n_cpu = cs.count_use_cpu_lora
        say("cold start: pipelined load, all layers on the GPU path")
        cs.admit([1, 0], tkn, mode="pipelined")
        ys3 = [[y.clone() for y in layer] for layer in y0]
        for layer in range(L):
            path = cs.start_layer(xs[layer], layer)
            assert path == "gpu"
            cs.finish_layer(path, xs[layer], layer, ys3[layer])
        torch.cuda.synchronize()
        assert cs.count_use_cpu_lora == n_cpu
        for layer in (0, 1, 2, 15, 31):
            for q, p in enumerate(NAMES):
                want = _expected("gpu", weights, [1, 0], scalings, tkn, layer, p, _bits(xs[layer]), _bits(y0[layer][q]))
                err = np.abs(ys3[layer][q].float().cpu().numpy() - want)
                assert np.all(err <= ATOL + RTOL * np.abs(want)), (layer, p, float(err.max()))
        served, rejected = cs.stop_workers()
        assert rejected == 0 and served == 3 * 2 * 3 * (3 + 3)       # projections x requests x chunks x CPU-served layers
    finally:
        cs.stop_workers()
        cpu.close()


def test_cold_start_free_running():
    """No forced wait: whatever mix of paths the timing gives, all 32 layers are served and every one is right."""
    pool, cpu, cs, weights = _setup(1)
    scalings = {0: 2.0}
    adapter_ids, tkn = [0], 64                                     # the reference's shape of a cold request: 64 tokens, 8 per worker
    gen = torch.Generator(device="cuda").manual_seed(5)
    xs = [torch.randn(tkn, H, device="cuda", generator=gen).half() for _ in range(L)]
    y0 = [[torch.randn(tkn, H, device="cuda", generator=gen).half() for _ in NAMES] for _ in range(L)]
    ys = [[y.clone() for y in layer] for layer in y0]
    try:
        say("cold start: free-running 32 layers")
        cs.admit(adapter_ids, tkn, mode="cpu_assisted")
        paths = []
        for layer in range(L):
            path = cs.start_layer(xs[layer], layer)
            cs.finish_layer(path, xs[layer], layer, ys[layer])
            paths.append(path)
        torch.cuda.synchronize()
        assert cs.count_use_cpu_lora + cs.count_use_gpu_lora == L
        for layer in range(0, L, 3):
            for q, p in enumerate(NAMES):
                want = _expected(paths[layer], weights, adapter_ids, scalings, tkn, layer, p, _bits(xs[layer]), _bits(y0[layer][q]))
                if paths[layer] == "cpu":
                    assert np.array_equal(_bits(ys[layer][q]), want), (layer, p)
                else:
                    err = np.abs(ys[layer][q].float().cpu().numpy() - want)
                    assert np.all(err <= ATOL + RTOL * np.abs(want)), (layer, p, float(err.max()))
    finally:
        cs.stop_workers()
        cpu.close()


def test_cold_start_next_batch_while_the_load_is_in_flight():
    """A second batch on an adapter whose load an earlier batch started depends on that load too: it may not read the
    pool before the rows are in (forced GPU path: the launch waits on the device; cached: the host waits).  A batch
    that needs a slot when none is free says so."""
    pool, cpu, cs, weights = _setup(5)
    scalings = {a: (2.0 if a % 2 == 0 else 0.5) for a in range(5)}
    tkn = 8
    gen = torch.Generator(device="cuda").manual_seed(11)
    x = torch.randn(tkn, H, device="cuda", generator=gen).half()
    y0 = [torch.randn(tkn, H, device="cuda", generator=gen).half() for _ in NAMES]
    gate_host = torch.empty(1 << 29, dtype=torch.uint8, pin_memory=True)
    gate_dev = torch.empty(1 << 29, dtype=torch.uint8, device="cuda")
    try:
        torch.cuda.synchronize()
        with torch.cuda.stream(cs.loader.stream):
            for _ in range(4):
                gate_dev.copy_(gate_host, non_blocking=True)
        say("cold start: two batches on one load")
        cs.admit([0], tkn, mode="cpu_assisted")
        cs.admit([0], tkn, mode="cpu_assisted")                    # same adapter again, its load still queued behind the gate
        assert len(cs.tickets) == 1 and not cs.use_gpu_pipeline(20)
        ys = [y.clone() for y in y0]
        cs.finish_layer(cs.start_layer(x, 20, force="gpu"), x, 20, ys)     # the launch waits on the device for layer 20's rows
        cs.admit([0], tkn, mode="cached")                          # the host waits for the rest of the load
        assert cs.tickets == [] and cs.use_gpu_pipeline(0)
        ys2 = [y.clone() for y in y0]
        cs.finish_layer(cs.start_layer(x, 3), x, 3, ys2)
        torch.cuda.synchronize()
        for layer, out in ((20, ys), (3, ys2)):
            for q, p in enumerate(NAMES):
                want = _expected("gpu", weights, [0], scalings, tkn, layer, p, _bits(x), _bits(y0[q]))
                err = np.abs(out[q].float().cpu().numpy() - want)
                assert np.all(err <= ATOL + RTOL * np.abs(want)), (layer, p, float(err.max()))
        cs.admit([1, 2, 3], tkn, mode="on_demand")                 # the pool has four slots
        with pytest.raises(RuntimeError, match="no free slot"):
            cs.admit([4], tkn, mode="on_demand")
        cs.evict(2)
        cs.admit([4], tkn, mode="on_demand")
        ys3 = [y.clone() for y in y0]
        cs.finish_layer(cs.start_layer(x, 31), x, 31, ys3)
        torch.cuda.synchronize()
        want = _expected("gpu", weights, [4], scalings, tkn, 31, "v", _bits(x), _bits(y0[2]))
        err = np.abs(ys3[2].float().cpu().numpy() - want)
        assert np.all(err <= ATOL + RTOL * np.abs(want))
        with pytest.raises(KeyError):
            cs.admit([7], tkn)
    finally:
        cs.stop_workers()
        cpu.close()
