"""GPU: decode steps of a replay of the reference's arrival trace (adapter per request from its popularity vector),
with adapters swapped into a pool smaller than the adapter population, against the oracle."""
import os

import numpy as np
import pytest
import torch

from gpu_common import assert_close_bits, say
from helpers import FP16, torch_to_bits
from mlora import trace_driver as td
from mlora import workloads
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def test_trace_steps_against_the_oracle():
    times = np.load(os.path.join(GOLDEN, "maf_trace_512.npy"), allow_pickle=False)
    pop = np.load(os.path.join(GOLDEN, "maf_popularity_128.npy"), allow_pickle=False)
    ids = workloads.draw_lora_ids(pop, len(times), seed=0)
    lens = td.draw_output_lengths(len(times), mean=48.0, seed=2)
    steps = td.simulate(times, ids, lens, step_s=0.03, running_max_req_size=24, max_prefill_batch_size=4, max_steps=500)
    decode = [s for s in steps if s.kind == "decode" and len(s.lora_ids) > 0]
    L, H, r, n_slots = 2, 256, 8, 16
    run = td.TraceRunner(L, H, r, n_slots, device="cuda", max_batch=32, seed=3)
    checked = loads_seen = 0
    last_size = -1
    for i, s in enumerate(decode):
        if len(set(s.lora_ids.tolist())) > n_slots:
            continue
        before = run.residency.loads
        # check a step when its batch differs from the last checked one or it had to swap adapters in
        check = checked < 6 and (run.residency.loads == 0 or len(s.lora_ids) != last_size)
        slots, ys = run.decode_step(s.lora_ids, accumulate=not check)
        swapped = run.residency.loads - before
        loads_seen += swapped
        if not check:
            continue
        torch.cuda.synchronize()
        T = len(s.lora_ids)
        say(f"trace step {s.index}: {T} requests, {len(set(s.lora_ids.tolist()))} adapters, {swapped} swapped in")
        pool = run.pool
        for layer in (0, L - 1):
            x = torch_to_bits(run.x[layer][:T])
            for pi, p in enumerate("qkv"):
                a_rows = torch_to_bits(pool.a_rows[p][layer])
                b_rows = torch_to_bits(pool.b_rows[p][layer])
                want = orc.lora_apply_paged(x, a_rows, b_rows, slots, pool.h_page_tbl, pool.h_page_tbl, pool.h_rank,
                                            pool.h_scaling, pool.page_rows, FP16)
                assert_close_bits(torch_to_bits(ys[layer][pi][:T]), want, FP16, f"step {s.index} layer {layer} {p}")
        # what sits on the slot's pages is the adapter the step asked for
        for a in set(s.lora_ids.tolist()):
            A, B = run.adapter_weights(a)["k"]
            rows = pool.rows_of(run.residency.slot_of[a])
            assert torch.equal(pool.a_rows["k"][1][rows].cpu(), A[1].t().half())
            assert torch.equal(pool.b_rows["k"][1][rows].cpu(), B[1].half())
        checked += 1
        last_size = T
        if checked >= 6 and loads_seen > n_slots and run.residency.evictions > 0:
            break
    assert checked >= 3 and run.residency.evictions > 0, (checked, run.residency.loads, run.residency.evictions)
