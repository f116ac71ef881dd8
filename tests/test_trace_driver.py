"""Trace-driven workload: the reference's arrival traces (data fixtures), its admission rule restated, and the
adapter residency bookkeeping -- host logic only."""
import os

import numpy as np
import pytest

from mlora import trace_driver as td
from mlora import workloads

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


@pytest.mark.parametrize("n,count", [(128, 434), (256, 1043), (512, 2231)])
def test_trace_fixtures(n, count):
    t = np.load(os.path.join(GOLDEN, f"maf_trace_{n}.npy"), allow_pickle=False)
    assert t.dtype == np.float64 and t.shape == (count,)
    assert np.all(np.diff(t) >= 0) and t[0] > 0 and t[-1] == 288.0
    # the traces are named after their adapter count; the arrival rate grows with it (about 1.5, 3.6 and 7.7 per second)
    assert abs(count / t[-1] - {128: 1.5, 256: 3.6, 512: 7.7}[n]) < 0.1


def test_parse_trace_reads_what_follows_the_separator(tmp_path):
    p = tmp_path / "t.txt"
    p.write_text("Number of Events: 3, Duration: 30, Rate: 6\n==========\n0.154\n0.285\n\n1.5\n")
    assert td.parse_trace(str(p)).tolist() == [0.154, 0.285, 1.5]
    p.write_text("0.1\n0.2\n")                               # no separator: nothing counts (client_maf.py:24-29)
    assert td.parse_trace(str(p)).size == 0


def test_simulate_follows_the_admission_rule():
    """Brute-force bookkeeping of a small replay: arrival order, at most `max_prefill_batch_size` admissions per
    step, never more than `running_max_req_size` running, one token per running request and decode step."""
    rng = np.random.default_rng(0)
    n = 60
    times = np.sort(rng.uniform(0, 3.0, n))
    ids = rng.integers(0, 9, n)
    lens = rng.integers(1, 12, n)
    steps = td.simulate(times, ids, lens, step_s=0.05, running_max_req_size=7, max_prefill_batch_size=3)
    admitted_order, decoded = [], np.zeros(n, int)
    running = []
    for s in steps:
        assert s.time >= 0 and s.kind in ("prefill", "decode")
        if s.kind == "prefill":
            assert 1 <= len(s.admitted) <= 3
            assert all(times[rq] <= s.time + 1e-12 for rq in s.admitted)
            admitted_order += s.admitted
            running += [rq for rq in s.admitted if lens[rq] > 1]
            assert len(running) <= 7
        else:
            assert len(s.lora_ids) == len(running) and len(running) > 0
            assert s.lora_ids.tolist() == [int(ids[rq]) for rq in running]
            for rq in running:
                decoded[rq] += 1
            running = [rq for rq in running if decoded[rq] < lens[rq] - 1]
    assert admitted_order == list(range(n))                    # first come, first served; everybody is served
    assert np.array_equal(decoded, np.maximum(lens - 1, 0)) and not running
    # a prefill step happens whenever somebody waits and there is room: no decode step leaves an arrived request outside
    assert len(td.simulate(times, ids, lens, max_steps=5)) == 5


def test_simulate_on_the_reference_trace_gives_changing_batches():
    times = np.load(os.path.join(GOLDEN, "maf_trace_128.npy"), allow_pickle=False)
    pop = np.load(os.path.join(GOLDEN, "maf_popularity_128.npy"), allow_pickle=False)
    ids = workloads.draw_lora_ids(pop, len(times), seed=0)
    lens = td.draw_output_lengths(len(times), mean=64.0, seed=1)
    assert lens.min() >= 1 and 40 < lens.mean() < 90
    steps = td.simulate(times, ids, lens, step_s=0.03, running_max_req_size=32, max_prefill_batch_size=4)
    dec = [s for s in steps if s.kind == "decode"]
    sizes = np.array([len(s.lora_ids) for s in dec])
    assert sizes.max() <= 32 and sizes.max() >= 4 and len(set(sizes.tolist())) > 3
    assert sum(len(s.admitted) for s in steps) == len(times)
    assert sizes.sum() == int(np.maximum(lens - 1, 0).sum())


def test_adapter_residency_is_lru_and_never_evicts_what_the_step_needs():
    r = td.AdapterResidency(3)
    assert [(a, e) for a, _, e in r.ensure([5, 7, 5])] == [(5, None), (7, None)]
    assert r.ensure([7]) == []
    todo = r.ensure([9, 5])                                   # 9 takes the last free slot, 5 is refreshed
    assert [(a, e) for a, _, e in todo] == [(9, None)]
    todo = r.ensure([1])                                      # least recently used is 7
    assert [(a, e) for a, _, e in todo] == [(1, 7)] and 7 not in r.slot_of
    todo = r.ensure([9, 5, 7])                                # 1 must go, never 9 or 5 (needed now)
    assert [(a, e) for a, _, e in todo] == [(7, 1)]
    assert sorted(r.slot_of.values()) == [0, 1, 2] and r.loads == 5 and r.evictions == 2
    assert r.slots(np.array([5, 7, 7, 9])).tolist() == [r.slot_of[5], r.slot_of[7], r.slot_of[7], r.slot_of[9]]
    with pytest.raises(MemoryError):
        r.ensure([1, 2, 3, 4])
