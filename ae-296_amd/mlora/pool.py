"""Paged, heterogeneous-rank adapter pool resident in HBM.

The reference keeps one dense tensor per projection and side, sized for a fixed rank
(``lightllm/models/lora_gpu.py:33-40``: ``{q,k,v}_down [N, L, r, Hin]``,
``{q,k,v}_up [N, L, Hout, r]``) and moves whole adapters with tensor copies
(``:165-188,202-217,229-242``).  Here an adapter of rank r owns ceil(r / page_rows)
pages of ``page_rows`` rank rows; the same page ids are used in every layer and
projection, so loading, evicting or re-ranking an adapter is a page-table update and
the kernels read the rows in place.

Layout in HBM, per projection p (Hin_p -> Hout_p) and layer l:
    a_rows[p][l] : [n_pages * page_rows, Hin_p]   rank rows of A^T
    b_rows[p][l] : [n_pages * page_rows, Hout_p]  rank rows of B
    page_tbl     : int32 [n_slots, max_pages]     (-1 = unused)
    rank         : int32 [n_slots]
    scaling      : float [n_slots]                (alpha / r)
"""
from __future__ import annotations

from typing import Dict, Sequence, Tuple

import numpy as np
import torch

from . import _ext


class AdapterPool:
    def __init__(self, n_layers: int, projections: Dict[str, Tuple[int, int]], n_slots: int, n_pages: int,
                 page_rows: int = 8, max_rank: int = 64, dtype: torch.dtype = torch.float16,
                 device: str | torch.device = "cuda"):
        if page_rows < 1 or page_rows > 64 or page_rows & (page_rows - 1):
            raise ValueError("page_rows must be a power of two in 1..64")
        if not 1 <= max_rank <= _ext.MAX_RANK:
            raise ValueError(f"max_rank must be in 1..{_ext.MAX_RANK}")
        for name, (hin, hout) in projections.items():
            if hin % 8 or hout % 8:
                raise ValueError(f"projection {name}: widths must be multiples of 8")
        self.n_layers = n_layers
        self.projections = dict(projections)
        self.n_slots = n_slots
        self.n_pages = n_pages
        self.page_rows = page_rows
        self.max_rank = max_rank
        self.max_pages = (max_rank + page_rows - 1) // page_rows
        self.dtype = dtype
        self.dtype_code = _ext.dtype_code(dtype)
        self.device = torch.device(device)
        n_rows = n_pages * page_rows
        self.a_rows = {p: torch.zeros((n_layers, n_rows, hin), dtype=dtype, device=self.device)
                       for p, (hin, _) in projections.items()}
        self.b_rows = {p: torch.zeros((n_layers, n_rows, hout), dtype=dtype, device=self.device)
                       for p, (_, hout) in projections.items()}
        # host mirrors are the source of truth; device copies are refreshed by sync()
        self.h_page_tbl = np.full((n_slots, self.max_pages), -1, np.int32)
        self.h_rank = np.zeros(n_slots, np.int32)
        self.h_scaling = np.zeros(n_slots, np.float32)
        self.page_tbl = torch.full((n_slots, self.max_pages), -1, dtype=torch.int32, device=self.device)
        self.rank = torch.zeros(n_slots, dtype=torch.int32, device=self.device)
        self.scaling = torch.zeros(n_slots, dtype=torch.float32, device=self.device)
        self._free = list(range(n_pages - 1, -1, -1))
        self._dirty = False
        self._call_args = {}       # (layer, projections) -> argument arrays of the decode call (kept by ops.bgmv)

    # ------------------------------------------------------------------ page table
    def allocate(self, slot: int, rank: int, scaling: float, pages: Sequence[int] | None = None) -> np.ndarray:
        """Give `slot` an adapter of the given rank; returns its page ids."""
        if not 0 <= slot < self.n_slots:
            raise IndexError(f"slot {slot} outside [0, {self.n_slots})")
        if not 1 <= rank <= self.max_rank:
            raise ValueError(f"rank {rank} outside 1..{self.max_rank}")
        if self.h_rank[slot] != 0:
            self.release(slot)
        need = (rank + self.page_rows - 1) // self.page_rows
        if pages is None:
            if need > len(self._free):
                raise MemoryError(f"adapter pool full: {need} pages needed, {len(self._free)} free")
            pages = [self._free.pop() for _ in range(need)]
        else:
            pages = list(pages)
            if len(pages) != need:
                raise ValueError(f"rank {rank} needs {need} pages, got {len(pages)}")
            taken = set(pages)
            if len(taken) != need or any(p < 0 or p >= self.n_pages for p in pages):
                raise ValueError("page ids must be distinct and inside the pool")
            free = set(self._free)
            if not taken <= free:
                raise ValueError("some requested pages are already in use")
            self._free = [p for p in self._free if p not in taken]
        self.h_page_tbl[slot, :] = -1
        self.h_page_tbl[slot, :need] = pages
        self.h_rank[slot] = rank
        self.h_scaling[slot] = scaling
        self._dirty = True
        return self.h_page_tbl[slot, :need].copy()

    def release(self, slot: int) -> None:
        """Evict the adapter in `slot` (the reference's remove_lora, lora_gpu.py:229-242, without copies)."""
        if not 0 <= slot < self.n_slots:
            raise IndexError(f"slot {slot} outside [0, {self.n_slots})")
        need = (int(self.h_rank[slot]) + self.page_rows - 1) // self.page_rows
        self._free.extend(int(p) for p in self.h_page_tbl[slot, :need][::-1])
        self.h_page_tbl[slot, :] = -1
        self.h_rank[slot] = 0
        self.h_scaling[slot] = 0.0
        self._dirty = True

    def move(self, src: int, dst: int) -> None:
        """Re-bind an adapter to another slot (the reference's merge_lora_prefill, lora_gpu.py:202-217,
        copies every layer's weights; here only the table rows move).  An adapter already in `dst` is
        evicted; `src` must hold one and differ from `dst`."""
        for name, slot in (("src", src), ("dst", dst)):
            if not 0 <= slot < self.n_slots:
                raise IndexError(f"{name} slot {slot} outside [0, {self.n_slots})")
        if src == dst:
            raise ValueError(f"move({src}, {dst}): source and destination are the same slot")
        if self.h_rank[src] == 0:
            raise ValueError(f"move: slot {src} holds no adapter")
        if self.h_rank[dst] != 0:
            self.release(dst)
        self.h_page_tbl[dst] = self.h_page_tbl[src]
        self.h_rank[dst] = self.h_rank[src]
        self.h_scaling[dst] = self.h_scaling[src]
        self.h_page_tbl[src, :] = -1
        self.h_rank[src] = 0
        self.h_scaling[src] = 0.0
        self._dirty = True

    def sync(self) -> None:
        """Push the host page table / rank / scaling to the device copies the kernels read."""
        if self._dirty:
            self.page_tbl.copy_(torch.from_numpy(self.h_page_tbl))
            self.rank.copy_(torch.from_numpy(self.h_rank))
            self.scaling.copy_(torch.from_numpy(self.h_scaling))
            self._dirty = False

    @property
    def free_pages(self) -> int:
        return len(self._free)

    # ------------------------------------------------------------------ weights
    def rows_of(self, slot: int) -> torch.Tensor:
        """Row indices (into a rows slab) of the adapter's rank rows, in rank order."""
        r = int(self.h_rank[slot])
        j = np.arange(r)
        rows = self.h_page_tbl[slot, j // self.page_rows].astype(np.int64) * self.page_rows + j % self.page_rows
        return torch.from_numpy(rows).to(self.device)

    def load(self, slot: int, layer: int, proj: str, A: torch.Tensor, B: torch.Tensor) -> None:
        """Write one (layer, projection) of an adapter: A is [Hin, r] (down), B is [r, Hout] (up)."""
        r = int(self.h_rank[slot])
        hin, hout = self.projections[proj]
        if tuple(A.shape) != (hin, r) or tuple(B.shape) != (r, hout):
            raise ValueError(f"expected A [{hin}, {r}] and B [{r}, {hout}], got {tuple(A.shape)} and {tuple(B.shape)}")
        rows = self.rows_of(slot)
        self.a_rows[proj][layer].index_copy_(0, rows, A.t().to(self.device, self.dtype).contiguous())
        self.b_rows[proj][layer].index_copy_(0, rows, B.to(self.device, self.dtype).contiguous())

    def slab_ptrs(self, layer: int, proj: str) -> Tuple[int, int]:
        return self.a_rows[proj][layer].data_ptr(), self.b_rows[proj][layer].data_ptr()
