"""Adapter swap-in: host (pinned) -> HBM pages, layer by layer, with per-layer readiness.

The reference loads an adapter for a new request by copying whole per-layer tensors from
pageable host memory into slot ``j`` of six dense GPU tensors, one copy and one slice assignment
per layer and tensor, in a separate swapper process that publishes a coarse progress code in
shared memory (``shared_tensor.py:111-154``: layers 8..31 first, code 2 after layer 15, 3 after 23,
4 after 31, then layers 0..7 and code 0); the model process polls that code per layer
(``lightllm/models/lora_gpu.py:298-321``) and the in-process variant rebuilds the tensors with
``torch.cat`` (``lora_gpu.py:165-188``).

Here an adapter is staged once in pinned host memory, layer-major; a load allocates the slot's
pages (a page-table update), then for each group of layers issues one host->device copy into a
staging buffer and scatter launches (as many layers per launch as the job table holds) that place the rank rows on the slot's pages
(``mlora_pool_scatter``), all on a copy stream of default priority, with an event per group.  A
consumer asks ``ticket.ready(layer)`` (event query, no synchronisation) or makes its own stream
wait for exactly the layers it is about to read (``ticket.wait_layer``).
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _ext
from .pool import AdapterPool

_VoidArr = C.c_void_p * _ext.SCATTER_MAX_JOBS
_IntArr = C.c_int32 * _ext.SCATTER_MAX_JOBS


@dataclass
class HostAdapter:
    """One adapter in pinned host memory: ``blob[l]`` holds, for every projection in pool order,
    the rank rows of A ([r, Hin]) followed by the rank rows of B ([r, Hout])."""
    rank: int
    scaling: float
    blob: torch.Tensor                       # [n_layers, layer_elems], pool dtype, pinned
    offsets: Dict[str, Tuple[int, int]]      # projection -> (element offset of A rows, of B rows) within a layer

    @property
    def nbytes(self) -> int:
        return self.blob.numel() * self.blob.element_size()


def layer_order(n_layers: int, first_layer: int) -> List[int]:
    """Load order of the reference's swapper (``shared_tensor.py:117,140``): ``first_layer`` .. L-1,
    then 0 .. ``first_layer``-1 (the early layers are the ones the CPU-assisted path covers meanwhile)."""
    first_layer = max(0, min(first_layer, n_layers))
    return list(range(first_layer, n_layers)) + list(range(0, first_layer))


@dataclass
class LoadTicket:
    slot: int
    order: List[int]                         # layers in load order
    group_of_layer: Dict[int, int]
    events: List[torch.cuda.Event] = field(default_factory=list)

    def ready(self, layer: int) -> bool:
        """True once the rows of `layer` are in the pool (never blocks)."""
        return self.events[self.group_of_layer[layer]].query()

    def wait_layer(self, layer: int, stream: Optional[torch.cuda.Stream] = None) -> None:
        """Make `stream` (default: the current one) wait on the device for `layer`; the host goes on."""
        (stream or torch.cuda.current_stream()).wait_event(self.events[self.group_of_layer[layer]])

    def wait(self) -> None:
        """Block the host until the whole adapter is loaded."""
        self.events[-1].synchronize()

    def layers_ready(self) -> int:
        return sum(1 for layer in self.order if self.ready(layer))

    def progress(self) -> int:
        """The reference's progress code for a 32-layer model generalised to L layers
        (``shared_tensor.py:128-136,148``): 1 = started, 2 / 3 / 4 = the second / third / fourth quarter
        of the layers is in, 0 = everything is in."""
        n = len(self.order)
        if all(self.ready(layer) for layer in self.order):
            return 0
        code = 1
        for c, last in ((2, n // 2 - 1), (3, 3 * n // 4 - 1), (4, n - 1)):
            if 0 <= last and self.ready(last):
                code = c
        return code

    def use_gpu_pipeline(self, layer_id: int) -> bool:
        """``Lora_GPU.use_gpu_pipeline`` (``lora_gpu.py:301-321``) with per-layer instead of per-quarter truth."""
        return self.ready(layer_id)


class AdapterLoader:
    def __init__(self, pool: AdapterPool, layers_per_copy: int = 8, first_layer: int = 8):
        if 2 * len(pool.projections) > _ext.SCATTER_MAX_JOBS:
            raise ValueError(f"at most {_ext.SCATTER_MAX_JOBS // 2} projections per pool")
        self.pool = pool
        self.layers_per_copy = max(1, int(layers_per_copy))
        self.first_layer = first_layer
        self.projs = list(pool.projections)
        self.stream = torch.cuda.Stream(device=pool.device)           # default priority
        self._stage_elems = pool.max_rank * sum(hin + hout for hin, hout in pool.projections.values())
        # one staging area for a whole adapter: copies and scatters run in order on one stream, so the
        # next load reuses it safely without any host-side wait
        self._staging = torch.empty((pool.n_layers, self._stage_elems), dtype=pool.dtype, device=pool.device)

    # ------------------------------------------------------------------ host side
    def layout(self, rank: int) -> Tuple[Dict[str, Tuple[int, int]], int]:
        off, offsets = 0, {}
        for p in self.projs:
            hin, hout = self.pool.projections[p]
            offsets[p] = (off, off + rank * hin)
            off += rank * (hin + hout)
        return offsets, off

    def stage(self, weights: Dict[str, Tuple[torch.Tensor, torch.Tensor]], rank: int, scaling: float) -> HostAdapter:
        """Copy an adapter into pinned host memory.  ``weights[p] = (A, B)`` with A ``[L, Hin, r]``
        (down) and B ``[L, r, Hout]`` (up), any device, any float dtype."""
        pool = self.pool
        offsets, layer_elems = self.layout(rank)
        blob = torch.empty((pool.n_layers, layer_elems), dtype=pool.dtype, pin_memory=True)
        for p in self.projs:
            hin, hout = pool.projections[p]
            A, B = weights[p]
            if tuple(A.shape) != (pool.n_layers, hin, rank) or tuple(B.shape) != (pool.n_layers, rank, hout):
                raise ValueError(f"projection {p}: expected A [{pool.n_layers}, {hin}, {rank}] and B "
                                 f"[{pool.n_layers}, {rank}, {hout}], got {tuple(A.shape)} and {tuple(B.shape)}")
            a0, b0 = offsets[p]
            blob[:, a0:a0 + rank * hin].copy_(A.transpose(1, 2).reshape(pool.n_layers, rank * hin))
            blob[:, b0:b0 + rank * hout].copy_(B.reshape(pool.n_layers, rank * hout))
        return HostAdapter(rank, float(scaling), blob, offsets)

    # ------------------------------------------------------------------ device side
    def load_async(self, slot: int, host: HostAdapter, pages: Optional[Sequence[int]] = None,
                   first_layer: Optional[int] = None, layers_per_copy: Optional[int] = None) -> LoadTicket:
        """Bind `slot` to the adapter (page-table update) and start moving its rows into the pool.
        Returns at once; nothing on the caller's streams waits unless it asks the ticket to.  `first_layer` and
        `layers_per_copy` override the loader's own for this load (layer 0 first, in small groups, suits a consumer
        that walks the layers in order and waits for each: `ticket.wait_layer`)."""
        pool = self.pool
        per_copy = self.layers_per_copy if layers_per_copy is None else max(1, int(layers_per_copy))
        page_ids = pool.allocate(slot, host.rank, host.scaling, pages)
        pages_c = (C.c_int32 * len(page_ids))(*[int(v) for v in page_ids])
        order = layer_order(pool.n_layers, self.first_layer if first_layer is None else first_layer)
        ticket = LoadTicket(slot, order, {})
        layer_elems = host.blob.shape[1]
        lib = _ext.lib()
        esz = host.blob.element_size()
        self.stream.wait_stream(torch.cuda.current_stream())          # rows of an evicted adapter may still be in use
        with torch.cuda.stream(self.stream):
            for g0 in range(0, len(order), per_copy):
                group = order[g0:g0 + per_copy]
                # consecutive layers travel as one copy
                runs, start = [], 0
                for i in range(1, len(group) + 1):
                    if i == len(group) or group[i] != group[i - 1] + 1:
                        runs.append((group[start], group[i - 1] + 1))
                        start = i
                for l0, l1 in runs:
                    self._staging[l0:l1, :layer_elems].copy_(host.blob[l0:l1], non_blocking=True)
                # as many layers per scatter launch as the job table holds
                per_launch = max(1, _ext.SCATTER_MAX_JOBS // (2 * len(self.projs)))
                for i0 in range(0, len(group), per_launch):
                    src, dst, width = _VoidArr(), _VoidArr(), _IntArr()
                    n_jobs = 0
                    for layer in group[i0:i0 + per_launch]:
                        base = self._staging[layer].data_ptr()
                        for p in self.projs:
                            hin, hout = pool.projections[p]
                            a0, b0 = host.offsets[p]
                            a_ptr, b_ptr = pool.slab_ptrs(layer, p)
                            src[n_jobs], dst[n_jobs], width[n_jobs] = base + a0 * esz, a_ptr, hin
                            src[n_jobs + 1], dst[n_jobs + 1], width[n_jobs + 1] = base + b0 * esz, b_ptr, hout
                            n_jobs += 2
                    rc = lib.mlora_pool_scatter(n_jobs, src, dst, width, pages_c, len(page_ids), host.rank,
                                                pool.page_rows, pool.n_pages, esz, self.stream.cuda_stream)
                    _ext.check(rc)
                ev = torch.cuda.Event()
                ev.record(self.stream)
                for layer in group:
                    ticket.group_of_layer[layer] = len(ticket.events)
                ticket.events.append(ev)
        return ticket
