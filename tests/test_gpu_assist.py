"""GPU parity of the CPU-assist transport: hidden states reach the request slots bit for bit, every
worker is woken with its code, and the results come back as the rank's column slice -- with the CPU
checker standing in for the reference's worker processes (the package itself computes nothing on the
CPU)."""
import threading

import numpy as np
import pytest
import torch

from gpu_common import say
from mlora import Lora_CPU
from mlora.lora_cpu import PROMPT_MAX_LENGTH, chunk_of
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def _serve(cpu, down, up, stop, served):
    """Stand-in for lora_cpu/lora_shm_op/app.py:102-143: poll the signals, compute the chunk, reset."""
    while not stop.is_set():
        for q in range(3):
            for w in range(cpu.lora_num):
                code = int(cpu.np_signal[q, w])
                if code > 1:
                    row_id = code - (2 + 200 * q)
                    assert row_id == w
                    tkn = int(cpu.np_tkn_len[0])
                    req, t0, n = chunk_of(row_id, tkn, cpu.cpu_capacity)
                    x = np.ascontiguousarray(cpu.np_x[req, t0:t0 + n])
                    cpu.np_out[q][req, t0:t0 + n] = orc.cpu_lora_worker(x, down[q], up[q])
                    cpu.np_signal[q, w] = 0
                    served.append((q, w))


@pytest.mark.parametrize("batch,tkn,cap,tp,gpu_id", [(3, 20, 8, 2, 1), (2, 7, 16, 1, 0), (1, 256, 64, 4, 3)])
def test_assist_round_trip(batch, tkn, cap, tp, gpu_id):
    rng = np.random.default_rng(batch * 100 + tkn)
    H, r = 256, 8
    cfg = dict(batch_size=batch, lora_num=12, tp_degree=tp, hidden_dim=H, lora_rank=r, token_per_lora=cap, n_layers=2)
    cpu = Lora_CPU(cfg, gpu_id=gpu_id)
    try:
        down = [(rng.standard_normal((H, r)) * 0.05).astype(np.float32) for _ in range(3)]
        up = [(rng.standard_normal((r, H)) * 0.05).astype(np.float32) for _ in range(3)]
        hidden = torch.randn(batch * tkn, H, device="cuda", dtype=torch.float16)
        h_bits = hidden.cpu().numpy().view(np.uint16)
        stop, served = threading.Event(), []
        worker = threading.Thread(target=_serve, args=(cpu, down, up, stop, served), daemon=True)
        worker.start()
        say(f"assist: export batch={batch} tkn={tkn} cap={cap}")
        cpu.invoke_lora_async(hidden, tkn, layer_id=0)
        q, k, v = cpu.collect_qkv(tkn, batch, timeout_s=30.0)
        torch.cuda.synchronize()
        stop.set()
        worker.join(timeout=5)
        cpr = (tkn - 1) // cap + 1
        assert sorted(served) == sorted((p, w) for p in range(3) for w in range(batch * cpr))
        # the slots hold the hidden states bit for bit, request b at slot b, and nothing else was touched
        for b in range(batch):
            assert np.array_equal(cpu.np_x[b, :tkn], h_bits[b * tkn:(b + 1) * tkn])
            assert not cpu.np_x[b, tkn:].any()
        assert not cpu.np_x[batch:].any()
        # results: the rank's column slice of what the worker arithmetic gives for every request
        out = H // tp
        for p, got in enumerate((q, k, v)):
            assert got.shape == (batch, tkn, out)
            want = orc.cpu_lora_worker(h_bits, down[p], up[p]).reshape(batch, tkn, H)[:, :, out * gpu_id:out * (gpu_id + 1)]
            assert np.array_equal(got.cpu().numpy().view(np.uint16), want)
    finally:
        cpu.close()


@pytest.mark.parametrize("batch,tkn,cap,tp,gpu_id,threads", [(3, 20, 8, 2, 1, 4), (8, 64, 16, 1, 0, 8), (2, 256, 64, 4, 2, 3)])
def test_assist_end_to_end_with_the_in_process_workers(batch, tkn, cap, tp, gpu_id, threads):
    """Export -> the package's own host workers (libmlora_cpu.so thread pool) -> import, two batches in a row
    through the same slots, each against the oracle's worker arithmetic, bit for bit."""
    rng = np.random.default_rng(900 + batch * tkn)
    H, r, N = 512, 16, 5
    cfg = dict(batch_size=batch, lora_num=32, tp_degree=tp, hidden_dim=H, lora_rank=r, token_per_lora=cap, n_layers=2)
    cpu = Lora_CPU(cfg, gpu_id=gpu_id)
    try:
        down = [(rng.standard_normal((N, H, r)) * 0.05).astype(np.float32) for _ in range(3)]
        up = [(rng.standard_normal((N, r, H)) * 0.05).astype(np.float32) for _ in range(3)]
        slot_adapter = rng.integers(0, N, cpu.lora_num).astype(np.int32)
        cpu.start_workers(down, up, n_threads=threads, slot_adapter=slot_adapter)
        out = H // tp
        n_chunks = 0
        for rep, (b, t) in enumerate(((batch, tkn), (max(1, batch - 1), max(1, tkn // 2)))):
            hidden = torch.randn(b * t, H, device="cuda", dtype=torch.float16)
            h_bits = hidden.cpu().numpy().view(np.uint16).reshape(b, t, H)
            say(f"assist end to end: batch={b} tkn={t} cap={cap} threads={threads} (call {rep})")
            cpu.invoke_lora_async(hidden, t, layer_id=rep)
            res = cpu.collect_qkv(t, b, timeout_s=30.0)
            torch.cuda.synchronize()
            n_chunks += 3 * b * ((t - 1) // cap + 1)
            for p, got in enumerate(res):
                assert got.shape == (b, t, out)
                for i in range(b):
                    a = slot_adapter[i]
                    want = orc.cpu_lora_worker(np.ascontiguousarray(h_bits[i]), down[p][a], up[p][a])[:, out * gpu_id:out * (gpu_id + 1)]
                    assert np.array_equal(got[i].cpu().numpy().view(np.uint16), want), (rep, p, i)
        assert cpu.stop_workers() == (n_chunks, 0)
    finally:
        cpu.close()


def test_assist_rejects_what_does_not_fit():
    cfg = dict(batch_size=4, lora_num=4, tp_degree=1, hidden_dim=64, lora_rank=8, token_per_lora=8, n_layers=1)
    cpu = Lora_CPU(cfg)
    try:
        with pytest.raises(ValueError):
            cpu.invoke_lora_async(torch.zeros(3 * 20, 64, device="cuda", dtype=torch.float16), 20)   # 9 workers > 4
        with pytest.raises(ValueError):
            cpu.invoke_lora_async(torch.zeros(10, 32, device="cuda", dtype=torch.float16), 5)
        assert chunk_of(5, 20, 8) == (1, 16, 4) and chunk_of(0, 1, 8) == (0, 0, 1)
        assert PROMPT_MAX_LENGTH == 256
    finally:
        cpu.close()
