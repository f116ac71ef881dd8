"""Drive the decode kernels from the reference's request traces: arrival times, per-request adapter draws and
continuous batching, with adapters swapped into a pool that is smaller than the adapter population.

What is mirrored from the reference:

* arrival times: its trace files (``benchmark/traces/maf_trace_*_scale_0.4.txt``: one arrival time per line
  after a ``=====`` line, parsed as ``benchmark/client_maf.py:20-30`` parses them); the times are kept as data
  under ``tests/golden/maf_trace_*.npy``;
* the adapter of request i: the i-th draw of ``np.random.choice(N, p=popularity)`` after ``np.random.seed(0)``
  (``client_maf.py:41-42,53``; ``workloads.draw_lora_ids``);
* batching: every scheduler step first admits waiting requests in arrival order, at most
  ``max_prefill_batch_size`` of them and never beyond ``running_max_req_size`` running requests, and otherwise
  decodes one token for every running request (``lightllm/server/router/manager.py:142-300``,
  ``router/req_queue.py:67-113``); the per-request ``lora_id`` reaches the model as an int32 vector
  (``router/model_infer/pre_process.py:50,100``) -- which the reference then drops (``lora_gpu.py:120,124``)
  and this driver uses.

What is synthetic: output lengths (the reference takes them from a dataset that is not part of it,
``client_maf.py:33-34,50``) are drawn from a seeded geometric distribution; the virtual duration of a scheduler
step is a parameter.
"""
from __future__ import annotations

from collections import OrderedDict
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np


def parse_trace(path: str) -> np.ndarray:
    """Arrival times of a trace file in the reference's text format: everything after the ``=====`` line, one
    float per line (``benchmark/client_maf.py:20-30``)."""
    times, started = [], False
    with open(path) as f:
        for line in f:
            if "=======" in line:
                started = True
                continue
            if started and line.strip():
                times.append(float(line.strip()))
    return np.asarray(times, np.float64)


def draw_output_lengths(n: int, mean: float = 128.0, seed: int = 0, cap: int = 1024) -> np.ndarray:
    """Synthetic ``max_new_tokens`` per request: 1 + geometric with the given mean, capped."""
    rng = np.random.default_rng(seed)
    return np.minimum(1 + rng.geometric(1.0 / max(mean, 1.0), size=n), cap).astype(np.int32)


@dataclass
class TraceStep:
    """One scheduler step: `kind` is "prefill" (the requests in `admitted` join the batch) or "decode" (one token
    for every running request); `lora_ids` holds the adapter of every running request after the step's
    admissions, in admission order."""
    index: int
    time: float
    kind: str
    lora_ids: np.ndarray
    admitted: List[int] = field(default_factory=list)       # request numbers admitted in this step
    finished: int = 0


def simulate(event_times: Sequence[float], lora_ids: Sequence[int], out_lens: Sequence[int], step_s: float = 0.03,
             running_max_req_size: int = 256, max_prefill_batch_size: int = 8, max_steps: Optional[int] = None) -> List[TraceStep]:
    """Scheduler steps of a trace replay under the reference's admission rule.  Virtual time advances by `step_s`
    per step; when nothing runs and nothing waits it jumps to the next arrival."""
    n = len(event_times)
    if not (len(lora_ids) == len(out_lens) == n):
        raise ValueError("event_times, lora_ids and out_lens must have one entry per request")
    steps: List[TraceStep] = []
    running: "OrderedDict[int, int]" = OrderedDict()         # request -> tokens left
    nxt, t = 0, 0.0
    while (nxt < n or running) and (max_steps is None or len(steps) < max_steps):
        if not running and nxt < n and event_times[nxt] > t:
            t = float(event_times[nxt])
        waiting = 0
        while nxt + waiting < n and event_times[nxt + waiting] <= t:
            waiting += 1
        room = min(running_max_req_size - len(running), max_prefill_batch_size)
        if waiting > 0 and room > 0:
            admitted = list(range(nxt, nxt + min(waiting, room)))
            for rq in admitted:
                running[rq] = int(out_lens[rq]) - 1         # the prefill yields the first token
            nxt += len(admitted)
            done = [rq for rq in admitted if running[rq] <= 0]
            for rq in done:
                del running[rq]
            steps.append(TraceStep(len(steps), t, "prefill", np.array([lora_ids[rq] for rq in running], np.int32), admitted, len(done)))
        else:
            ids = np.array([lora_ids[rq] for rq in running], np.int32)
            done = []
            for rq in running:
                running[rq] -= 1
                if running[rq] <= 0:
                    done.append(rq)
            for rq in done:
                del running[rq]
            steps.append(TraceStep(len(steps), t, "decode", ids, [], len(done)))
        t += step_s
    return steps


class AdapterResidency:
    """Which adapter sits in which pool slot: a fixed number of slots, least recently used adapter evicted first,
    never one that the current step needs.  Pure bookkeeping (no GPU)."""

    def __init__(self, n_slots: int):
        self.n_slots = n_slots
        self.slot_of: "OrderedDict[int, int]" = OrderedDict()    # adapter -> slot, least recently used first
        self.free = list(range(n_slots - 1, -1, -1))
        self.loads = 0
        self.evictions = 0

    def ensure(self, needed: Sequence[int]) -> List[tuple]:
        """Make every adapter in `needed` resident.  Returns [(adapter, slot, evicted adapter or None)] for the
        ones that have to be loaded.  Raises if the step needs more distinct adapters than there are slots."""
        distinct = list(dict.fromkeys(int(a) for a in needed))
        if len(distinct) > self.n_slots:
            raise MemoryError(f"a step needs {len(distinct)} adapters, the pool has {self.n_slots} slots")
        keep = set(distinct)
        todo = []
        for a in distinct:
            if a in self.slot_of:
                self.slot_of.move_to_end(a)
                continue
            evicted = None
            if self.free:
                slot = self.free.pop()
            else:
                evicted = next(v for v in self.slot_of if v not in keep)
                slot = self.slot_of.pop(evicted)
                self.evictions += 1
            self.slot_of[a] = slot
            self.loads += 1
            todo.append((a, slot, evicted))
        return todo

    def slots(self, lora_ids: np.ndarray) -> np.ndarray:
        return np.array([self.slot_of[int(a)] for a in lora_ids], np.int32)


class TraceRunner:
    """Runs the decode steps of a simulated trace on the GPU: adapters are staged in pinned host memory on first
    use (weights drawn from a generator seeded by the adapter id), swapped into a paged pool of `n_slots` slots
    through ``AdapterLoader`` when a step needs them, and every decode step is one gather plus one BGMV call per
    layer over q, k, v (the projections the reference applies LoRA to)."""

    def __init__(self, n_layers: int, hidden: int, rank: int, n_slots: int, device="cuda", dtype=None, seed: int = 0,
                 scaling: float = 2.0, max_batch: int = 256):
        import torch

        from . import AdapterLoader, AdapterPool
        self.torch = torch
        self.n_layers, self.hidden, self.rank, self.scaling = n_layers, hidden, rank, scaling
        self.dtype = dtype or torch.float16
        self.device = torch.device(device)
        page_rows = 8
        self.pool = AdapterPool(n_layers, {p: (hidden, hidden) for p in "qkv"}, n_slots,
                                n_slots * ((rank + page_rows - 1) // page_rows), page_rows=page_rows, max_rank=rank,
                                dtype=self.dtype, device=self.device)
        self.loader = AdapterLoader(self.pool, layers_per_copy=n_layers, first_layer=0)
        self.residency = AdapterResidency(n_slots)
        self.host: Dict[int, object] = {}
        self.seed = seed
        gen = torch.Generator(device=self.device)
        gen.manual_seed(seed + 99)
        self.x = [torch.randn(max_batch, hidden, device=self.device, generator=gen).to(self.dtype) for _ in range(n_layers)]
        self.y = [[torch.zeros(max_batch, hidden, device=self.device, dtype=self.dtype) for _ in range(3)] for _ in range(n_layers)]
        self.max_batch = max_batch
        # the host runs ahead of the GPU: a ring of pinned index buffers, each reused only after its copy has run
        self._ring = [(torch.empty(max_batch, dtype=torch.int32, pin_memory=True),
                       torch.empty(max_batch, dtype=torch.int32, device=self.device), torch.cuda.Event()) for _ in range(8)]
        self._ring_at = 0
        self._plans: Dict[int, object] = {}
        self.tickets: List[object] = []

    def adapter_weights(self, adapter: int):
        """A [L, hidden, r] and B [L, r, hidden] of q, k, v for one adapter id (deterministic)."""
        torch = self.torch
        g = torch.Generator().manual_seed(self.seed * 1000003 + int(adapter))
        return {p: (torch.randn(self.n_layers, self.hidden, self.rank, generator=g) * 0.02,
                    torch.randn(self.n_layers, self.rank, self.hidden, generator=g) * 0.02) for p in "qkv"}

    def make_resident(self, lora_ids: np.ndarray) -> int:
        """Swap in what the step needs and is not in the pool; returns the number of adapters loaded."""
        todo = self.residency.ensure(lora_ids)
        for adapter, slot, _evicted in todo:
            if adapter not in self.host:
                self.host[adapter] = self.loader.stage(self.adapter_weights(adapter), self.rank, self.scaling)
            self.tickets.append(self.loader.load_async(slot, self.host[adapter]))
        if todo:
            # the decode launches of this step read every layer: the compute stream waits for the copy stream
            self.torch.cuda.current_stream().wait_stream(self.loader.stream)
            self.tickets.clear()
        return len(todo)

    def decode_step(self, lora_ids: np.ndarray, accumulate: bool = True):
        """One decode step for a batch whose requests use `lora_ids`; returns (tok_adapter slots, y tensors)."""
        from . import ops
        torch = self.torch
        T = len(lora_ids)
        if T == 0:
            return np.zeros(0, np.int32), None
        if T > self.max_batch:
            raise ValueError(f"batch of {T} exceeds the runner's max_batch {self.max_batch}")
        self.make_resident(lora_ids)
        slots = self.residency.slots(lora_ids)
        host, devbuf, ev = self._ring[self._ring_at]
        self._ring_at = (self._ring_at + 1) % len(self._ring)
        ev.synchronize()                                       # the launches that read this buffer eight steps ago are done
        host[:T].copy_(torch.from_numpy(slots))
        tok = devbuf[:T]
        tok.copy_(host[:T], non_blocking=True)
        plan = self._plans.get(T)
        plan = ops.plan_decode(tok, self.pool, out=plan) if plan is not None else ops.plan_decode(tok, self.pool)
        self._plans[T] = plan
        for l in range(self.n_layers):
            ys = [y[:T] for y in self.y[l]]
            xl = self.x[l][:T]
            ops.bgmv(ys, [xl, xl, xl], self.pool, l, ["q", "k", "v"], tok, plan=plan, accumulate=accumulate)
        ev.record()
        return slots, self.y
