"""Prefill while adapters are still loading: the per-layer switch between the CPU-assisted path and the GPU path.

What is mirrored from the reference (its subject: hiding an adapter's cold start):

* the router marks the new requests' adapters for loading and starts the prefill at once in ``aaas_mode="cpu_lora"``
  (``lightllm/server/router/manager.py:175-188``), while the swapper copies layers 8..L-1, then 0..7, into the pool
  (``shared_tensor.py:111-154``);
* every layer asks ``gpu_lora.use_gpu_pipeline(layer)`` (``lightllm/models/lora_gpu.py:298-321``) and serves q, k, v
  either on the GPU from the rows that have landed, or through ``cpu_lora.invoke_lora_async`` -- hidden states out to
  the host workers -- with the base projections running meanwhile and ``cpu_lora.collect_qkv`` +
  ``q += q_lora`` after them (``lightllm/models/llama/layer_infer/transformer_layer_infer.py:114-171``).

The three serving modes the reference compares (``README.md:86-89``) are the three ways ``admit`` can be called:
``cached`` (adapters already resident), ``cpu_assisted`` (load starts, prefill starts at once) and ``on_demand``
(prefill waits for the whole load).  A fourth, ``pipelined``, is this build's own: the load runs layer 0 first in
small groups and every layer's GPU work waits on the device for just its own group, so the host link is hidden
behind the layers themselves and no host worker is needed (on a link that moves an adapter in the time of a few
layers this is the fastest cold path).

Differences by design: readiness is per layer (an event per group of layers instead of the swapper's four progress
codes); the GPU path adds the delta into the base projection outputs in one SGMV call over q, k, v instead of three
``torch.bmm`` pairs and three adds; the host workers are threads of this process (``Lora_CPU.start_workers``).
Requests of a batch have the same number of tokens, as the reference's ``input.view(batch_size, -1, H)`` requires.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import ops
from .loader import AdapterLoader, HostAdapter, LoadTicket
from .lora_cpu import Lora_CPU
from .pool import AdapterPool

MODES = ("cached", "cpu_assisted", "on_demand", "pipelined")


class ColdStartPrefill:
    def __init__(self, pool: AdapterPool, cpu: Lora_CPU, max_adapters: int, names: Sequence[str] = ("q", "k", "v"),
                 layers_per_copy: int = 8, first_layer: int = 8):
        self.pool, self.cpu = pool, cpu
        self.names = list(names)
        if len(self.names) != 3:
            raise ValueError("the CPU-assisted path serves exactly three projections (q, k, v)")
        H = cpu.hidden_dim
        for p in self.names:
            if pool.projections[p] != (H, H):
                raise ValueError(f"projection {p} must be {H} -> {H} (the workers' slots are hidden_dim wide)")
        if cpu.tp_degree != 1:
            raise ValueError("tp_degree 1 only: the pool holds whole projections")
        self.loader = AdapterLoader(pool, layers_per_copy=layers_per_copy, first_layer=first_layer)
        self.max_adapters = max_adapters
        self.rank = pool.max_rank
        L = pool.n_layers
        # the workers' own copies of the adapters (fp32, as lora_cpu/lora_shm_op/app.py:38-45 keeps them), one entry per
        # (adapter, layer): entry a * L + l; `slot_adapter[b]` names the entry of request b for the layer in flight
        self.down = [np.zeros((max_adapters * L, H, self.rank), np.float32) for _ in self.names]
        self.up = [np.zeros((max_adapters * L, self.rank, H), np.float32) for _ in self.names]
        self.slot_adapter = np.zeros(cpu.lora_num, np.int32)
        self.host: Dict[int, HostAdapter] = {}
        self.resident: Dict[int, int] = {}            # adapter id -> pool slot
        self.tickets: List[LoadTicket] = []           # loads the batch in flight depends on
        self._loading: Dict[int, LoadTicket] = {}     # adapter id -> its load, until it is seen complete
        self.count_use_gpu_lora = 0                   # transformer_layer_infer.py:117-118
        self.count_use_cpu_lora = 0
        self._batch = None
        self._mode = None
        self._plan = None

    # ------------------------------------------------------------------ adapters
    def register_adapter(self, aid: int, weights: Dict[str, Tuple[torch.Tensor, torch.Tensor]], scaling: float) -> None:
        """``weights[p] = (A [L, H, r], B [L, r, H])``: staged once in pinned host memory for the loader, and copied
        (fp32, scaling folded into B) for the host workers."""
        if not 0 <= aid < self.max_adapters:
            raise IndexError(f"adapter id {aid} outside [0, {self.max_adapters})")
        L = self.pool.n_layers
        for p in self.names:
            if weights[p][0].shape[2] != self.rank:
                raise ValueError(f"adapters of this pool have rank {self.rank}")
        self.host[aid] = self.loader.stage(weights, self.rank, scaling)
        for q, p in enumerate(self.names):
            A, B = weights[p]
            # the values the pool will hold (rounded to the pool dtype), widened to fp32
            self.down[q][aid * L:(aid + 1) * L] = A.to(self.pool.dtype).float().cpu().numpy()
            self.up[q][aid * L:(aid + 1) * L] = (B.to(self.pool.dtype).float() * float(scaling)).cpu().numpy()

    def start_workers(self, n_threads: int) -> None:
        self.cpu.start_workers(self.down, self.up, n_threads=n_threads, slot_adapter=self.slot_adapter)

    def stop_workers(self):
        return self.cpu.stop_workers()

    def evict(self, aid: int) -> None:
        """Give the adapter's pages back.  A load of it that is still running finishes on the loader's stream first
        (the next load into these pages is queued behind it); no batch that uses the adapter may be in flight."""
        slot = self.resident.pop(aid, None)
        self._loading.pop(aid, None)
        if slot is not None:
            self.pool.release(slot)

    # ------------------------------------------------------------------ a batch
    def admit(self, adapter_ids: Sequence[int], tkn: int, mode: str = "cpu_assisted") -> None:
        """Start a prefill batch: request b uses adapter ``adapter_ids[b]`` and has ``tkn`` tokens.  Adapters that are
        not resident start loading (``cpu_assisted``: the layers go on at once; ``on_demand``: the host waits for
        the loads first; ``pipelined``: layer 0 is loaded first and every layer waits on the device for its own
        rows; ``cached``: every adapter must be resident)."""
        if mode not in MODES:
            raise ValueError(f"mode must be one of {MODES}")
        B = len(adapter_ids)
        self.tickets = []
        slots = []
        for b, aid in enumerate(adapter_ids):
            if aid not in self.host:
                raise KeyError(f"adapter {aid} was never registered")
            if aid in self.resident:
                slots.append(self.resident[aid])
                t = self._loading.get(aid)
                if t is not None:
                    # bound to a slot by an earlier batch and possibly still on its way: this batch depends on that load too
                    if t.progress() == 0:
                        del self._loading[aid]
                    elif t not in self.tickets:
                        self.tickets.append(t)
                continue
            if mode == "cached":
                raise RuntimeError(f"adapter {aid} is not resident")
            used = set(self.resident.values())
            slot = next((s for s in range(self.pool.n_slots) if s not in used), None)
            if slot is None:
                raise RuntimeError(f"no free slot for adapter {aid}: evict one of {sorted(self.resident)} first")
            order = dict(first_layer=0, layers_per_copy=2) if mode == "pipelined" else {}
            t = self.loader.load_async(slot, self.host[aid], **order)    # the router's progress = 1 (manager.py:178-181)
            self.tickets.append(t)
            self._loading[aid] = t
            self.resident[aid] = slot
            slots.append(slot)
        if mode in ("on_demand", "cached"):
            # on demand: the prefill starts when the adapters are in.  cached: they are, unless an earlier batch started
            # a load that has not finished -- then this one waits for it the same way
            for t in self.tickets:
                t.wait()
            for aid in adapter_ids:
                self._loading.pop(aid, None)
            self.tickets = []
        dev = self.pool.device
        seg_start = torch.arange(0, B * tkn, tkn, dtype=torch.int32, device=dev)
        seg_len = torch.full((B,), tkn, dtype=torch.int32, device=dev)
        seg_adapter = torch.tensor(slots, dtype=torch.int32, device=dev)
        self._plan = ops.plan_prefill(seg_start, seg_len, seg_adapter, B * tkn, self.pool, n_proj=len(self.names))
        self._batch = (list(adapter_ids), tkn)
        self._mode = mode

    def use_gpu_pipeline(self, layer: int) -> bool:
        """``Lora_GPU.use_gpu_pipeline`` (lora_gpu.py:301-321): the rows of this layer are in the pool for every
        adapter of the batch."""
        return all(t.use_gpu_pipeline(layer) for t in self.tickets)

    def start_layer(self, x: torch.Tensor, layer: int, force: Optional[str] = None) -> str:
        """Before the base projections of a layer: on the CPU-assisted path the hidden states leave for the host
        workers now (transformer_layer_infer.py:129-131).  Returns the path taken, ``"gpu"`` or ``"cpu"``
        (``force`` overrides the choice, for tests)."""
        adapter_ids, tkn = self._batch
        path = force or ("gpu" if (self._mode == "pipelined" or self.use_gpu_pipeline(layer)) else "cpu")
        if path == "gpu":
            for t in self.tickets:
                t.wait_layer(layer)               # orders the stream after the rows' arrival (already past, unless pipelined or forced)
            self.count_use_gpu_lora += 1
        else:
            L = self.pool.n_layers
            for b, aid in enumerate(adapter_ids):
                self.slot_adapter[b] = aid * L + layer
            self.cpu.invoke_lora_async(x, tkn, layer)
            self.count_use_cpu_lora += 1
        return path

    def finish_layer(self, path: str, x: torch.Tensor, layer: int, qkv: Sequence[torch.Tensor]) -> None:
        """After the base projections: ``q += q_lora`` etc. (transformer_layer_infer.py:149-171).  GPU path: one SGMV
        call that accumulates into q, k, v; CPU path: each projection is brought back and added as soon as its
        workers are done."""
        adapter_ids, tkn = self._batch
        if path == "gpu":
            ops.sgmv_multi(list(qkv), [x] * len(self.names), self.pool, layer, self.names, self._plan, accumulate=True)
            return
        for q, res in self.cpu.collect_each(tkn, len(adapter_ids)):
            qkv[q].add_(res.view(-1, self.cpu.out_size))
