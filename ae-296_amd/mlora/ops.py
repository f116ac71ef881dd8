"""Operator surface of the multi-LoRA apply path, on torch tensors in HBM.

Three levels, all thin wrappers over the C ABI (``include/mlora.h``):

* ``add_lora_bgmv`` -- signature-compatible stand-in for ``punica.ops.add_lora_bgmv`` as
  the reference calls it (``lightllm/models/lora_gpu.py:138,150,162``), on the reference's
  own pool layout; ``lora_prefill_ref`` likewise for the ``torch.bmm`` pair (``:127-128``).
* ``plan_decode`` / ``bgmv`` / ``sgmv`` -- the paged-pool kernels.
* ``lora_apply`` -- hidden states, per-token adapter index, pool, base projection output
  to accumulate into.

Every function launches on ``torch.cuda.current_stream()`` and returns without
synchronising.  Nothing here computes on the CPU.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from . import _ext
from .pool import AdapterPool

_VoidArr = C.c_void_p * _ext.MAX_PROJ
_IntArr = C.c_int32 * _ext.MAX_PROJ


def _need_cuda(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError("mlora kernels take device tensors; got a CPU tensor")


def _need_contig(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_contiguous():
            raise ValueError("mlora kernels take contiguous tensors")


# ---------------------------------------------------------------------- gather / grouping
@dataclass
class DecodePlan:
    """Device-side grouping of one decode batch by adapter (written by ``mlora_pool_gather``)."""
    tok_adapter: torch.Tensor      # int32 [T]
    group: int
    perm: torch.Tensor             # int32 [T]
    seg_start: torch.Tensor
    seg_len: torch.Tensor
    seg_adapter: torch.Tensor
    chunk_start: torch.Tensor
    chunk_len: torch.Tensor
    chunk_adapter: torch.Tensor
    counters: torch.Tensor         # int32 [8]: n_seg, n_valid, n_chunks, n_bad
    work: torch.Tensor             # int32 [work_cap(T), 80] decode work records in launch order
    row_off: Optional[torch.Tensor] = None   # int32 [T, max_pages]
    tok_rank: Optional[torch.Tensor] = None
    tok_scale: Optional[torch.Tensor] = None
    vws: Optional[torch.Tensor] = None       # uint8: fp32 intermediate of the two-launch decode form

    @property
    def T(self) -> int:
        return self.tok_adapter.numel()


_n_cus = {}


def n_cus(device=None) -> int:
    """Compute units of `device` (default: the current one), asked once per device; where no device is present
    (planning on a host without a GPU) the MI355X's 256."""
    if not torch.cuda.is_available():
        return 256
    idx = torch.cuda.current_device() if device is None else torch.device(device).index
    if idx is None:
        idx = torch.cuda.current_device()
    if idx not in _n_cus:
        _n_cus[idx] = int(torch.cuda.get_device_properties(idx).multi_processor_count)
    return _n_cus[idx]


def default_group(T: int) -> int:
    """Tokens of one adapter per decode work item when the caller does not say: 1 up to 64 tokens and
    2 up to 128 (the batch then fits one workgroup per compute unit and runs as the single fused launch,
    see `decode_fused`), 4 beyond (measured per call, three projections: 8.5 us at 64 tokens against
    9.9 for the two-launch form, 10.8 against 13.2 at 128, 20.5 against 20.9 with 2 at 256)."""
    return 1 if T <= 64 else 2 if T <= 128 else 4


def decode_fused(T: int, group: int, n_proj: int, n_slots: int) -> bool:
    """Form of a planned decode call when the caller does not say: the single fused launch while its
    work items, one 512-thread workgroup each, fit the device in one round (the call is then bound by
    the dependent loads of one workgroup, and a second launch only adds to that); the shrink and expand
    launches beyond, where spreading one item over many workgroups is what fills the memory system.
    The item count is the host's estimate: groups of two leave one odd item for about every other adapter."""
    if group > 2:
        return False
    items = T if group == 1 else (T + 1) // 2 + min(T, n_slots) // 2
    return items * n_proj <= n_cus()


def group_for(T: int, n_proj: int, n_slots: int) -> int:
    """Tokens per work item for calls of `n_proj` projections: `default_group(T)` while such a call runs as the
    fused launch; once it runs as the shrink + expand pair, 4 from 65 tokens on (config 3, 128 tokens x 7
    projections: 0.267 ms per step with 2, 0.260 with 4)."""
    g = default_group(T)
    return 4 if (T > 64 and not decode_fused(T, g, n_proj, n_slots)) else g


def plan_decode(tok_adapter: torch.Tensor, pool: AdapterPool, group: Optional[int] = None, per_token: bool = False,
                out: Optional[DecodePlan] = None, n_proj: Optional[int] = None) -> DecodePlan:
    """Index/offset gather for a decode batch: groups tokens by adapter (stable) and cuts the
    groups into work items of at most `group` tokens (1, 2, 4 or 8; default by batch size and, when the
    caller says how many projections its calls will carry (`n_proj`), by the launch form those take).  Pass
    `out` to reuse a plan's buffers (no allocation; safe under graph capture)."""
    _need_cuda(tok_adapter)
    if tok_adapter.dtype != torch.int32:
        raise TypeError("tok_adapter must be int32")
    _need_contig(tok_adapter)
    T = tok_adapter.numel()
    if group is None:
        group = out.group if out is not None else (default_group(T) if n_proj is None else group_for(T, n_proj, pool.n_slots))
    pool.sync()
    dev = tok_adapter.device
    if out is None:
        i32 = dict(dtype=torch.int32, device=dev)
        nseg = max(1, min(T, pool.n_slots))
        out = DecodePlan(tok_adapter, group, torch.empty(max(T, 1), **i32), torch.empty(nseg, **i32),
                         torch.empty(nseg, **i32), torch.empty(nseg, **i32), torch.empty(max(T, 1), **i32),
                         torch.empty(max(T, 1), **i32), torch.empty(max(T, 1), **i32),
                         torch.zeros(_ext.CNT_WORDS, **i32),
                         torch.empty((max(_ext.work_cap(T), 8), _ext.WORK_WORDS), **i32))
        if per_token:
            out.row_off = torch.empty((max(T, 1), pool.max_pages), **i32)
            out.tok_rank = torch.empty(max(T, 1), **i32)
            out.tok_scale = torch.empty(max(T, 1), dtype=torch.float32, device=dev)
    else:
        out.tok_adapter = tok_adapter
        out.group = group
    rc = _ext.lib().mlora_pool_gather(
        _ext.ptr(tok_adapter), T, _ext.ptr(pool.page_tbl), _ext.ptr(pool.rank), _ext.ptr(pool.scaling),
        pool.n_slots, pool.max_pages, pool.page_rows, pool.n_pages,
        _ext.ptr(out.row_off), _ext.ptr(out.tok_rank), _ext.ptr(out.tok_scale),
        _ext.ptr(out.perm), _ext.ptr(out.seg_start), _ext.ptr(out.seg_len), _ext.ptr(out.seg_adapter),
        _ext.ptr(out.chunk_start), _ext.ptr(out.chunk_len), _ext.ptr(out.chunk_adapter), group,
        _ext.ptr(out.counters), _ext.ptr(out.work), _ext.current_stream_ptr())
    _ext.check(rc)
    return out


# ---------------------------------------------------------------------- two halves of a mixed batch side by side
class SideStream:
    """A second stream (default priority) with its fork and join events.  The decode tokens and the prefill
    segments of a mixed batch touch different rows of x and y and only read the pool, so their launches need no
    order between them: `side_by_side` puts one half on this stream and joins before it returns, and each half's
    short tail of workgroups overlaps the other half's launches.  Works eagerly and under HIP graph capture (the
    fork and the join become graph edges)."""

    def __init__(self, device=None):
        self.stream = torch.cuda.Stream(device=device)
        self.fork = torch.cuda.Event()
        self.join = torch.cuda.Event()


def side_by_side(side: SideStream, on_side, on_main) -> None:
    """Run `on_side()` on the side stream and `on_main()` on the current stream, both after everything already
    queued on the current stream; what follows on the current stream waits for both.  The two callables must
    not share a plan's intermediate buffers (a decode plan and a prefill plan never do)."""
    main = torch.cuda.current_stream()
    side.fork.record(main)
    side.stream.wait_event(side.fork)
    try:
        with torch.cuda.stream(side.stream):
            on_side()
        on_main()
    finally:
        # joined also when a half raised: work already queued on the side stream stays ordered before what follows
        side.join.record(side.stream)
        main.wait_event(side.join)


# ---------------------------------------------------------------------- decode
def bgmv(ys: Sequence[torch.Tensor], xs: Sequence[torch.Tensor], pool: AdapterPool, layer: int,
         projs: Sequence[str], tok_adapter: torch.Tensor, plan: Optional[DecodePlan] = None,
         accumulate: bool = True, fused: Optional[bool] = None) -> None:
    """Decode LoRA apply for up to 8 projections of one layer:
    ys[p][t] (+)= scaling[a] * (xs[p][t] . A_{p,a}) . B_{p,a},  a = tok_adapter[t].

    With a plan the call runs as a shrink launch and an expand launch over column slices
    (``fused=False``) or as one fused launch (``fused=True``), by default whichever `decode_fused`
    names for the batch; without a plan it is always the fused launch with one token per work item.  The two-launch form keeps its fp32
    intermediate in a buffer owned by the plan, allocated on the first call that needs it (so
    run one call before capturing a HIP graph); calls that share a plan must therefore follow each
    other on one stream, not overlap on several."""
    n = len(projs)
    if not (len(ys) == len(xs) == n) or not 1 <= n <= _ext.MAX_PROJ:
        raise ValueError(f"need 1..{_ext.MAX_PROJ} projections with one y and one x each")
    _need_cuda(tok_adapter, *ys, *xs)
    _need_contig(tok_adapter, *ys, *xs)
    if tok_adapter.dtype != torch.int32:
        raise TypeError("tok_adapter must be int32")
    T = tok_adapter.numel()
    # the slab pointers and widths of a (layer, projections) pair never change: their argument arrays are kept
    key = (layer, tuple(projs))
    cached = pool._call_args.get(key)
    if cached is None:
        av, bv, hi, ho = _VoidArr(), _VoidArr(), _IntArr(), _IntArr()
        for i, p in enumerate(projs):
            hi[i], ho[i] = pool.projections[p]
            av[i], bv[i] = pool.slab_ptrs(layer, p)
        cached = pool._call_args[key] = (av, bv, hi, ho, max(hi[i] for i in range(n)))
    av, bv, hi, ho, max_hin = cached
    yv, xv = _VoidArr(), _VoidArr()
    for i in range(n):
        if xs[i].dtype != pool.dtype or ys[i].dtype != pool.dtype:
            raise TypeError(f"x and y must have the pool dtype {pool.dtype}")
        if xs[i].shape[0] != T or xs[i].shape[1] != hi[i] or ys[i].shape[0] != T or ys[i].shape[1] != ho[i] or xs[i].dim() != 2 or ys[i].dim() != 2:
            raise ValueError(f"projection {projs[i]}: expected x [{T}, {hi[i]}] and y [{T}, {ho[i]}], "
                             f"got {tuple(xs[i].shape)} and {tuple(ys[i].shape)}")
        yv[i], xv[i] = ys[i].data_ptr(), xs[i].data_ptr()
    pool.sync()
    if plan is not None and plan.T != T:
        raise ValueError("plan was built for a different batch size")
    if fused is None:
        fused = plan is None or decode_fused(T, plan.group, n, pool.n_slots)
    if not fused and plan is None:
        raise ValueError("the two-launch form needs a plan")
    ws, ws_bytes = None, 0
    if not fused:
        ws_bytes = _ext.lib().mlora_bgmv_workspace_bytes(n, T, max_hin, pool.max_rank)
        if plan.vws is None or plan.vws.numel() < ws_bytes:
            plan.vws = torch.empty(ws_bytes, dtype=torch.uint8, device=tok_adapter.device)
        ws = plan.vws
    rc = _ext.lib().mlora_bgmv_multi(
        n, yv, xv, av, bv, hi, ho, _ext.ptr(tok_adapter), T,
        _ext.ptr(pool.page_tbl), _ext.ptr(pool.rank), _ext.ptr(pool.scaling),
        pool.n_slots, pool.max_pages, pool.page_rows, pool.n_pages, pool.max_rank,
        _ext.ptr(plan.work) if plan else None, plan.group if plan else 1,
        _ext.ptr(ws), ws_bytes,
        pool.dtype_code, int(accumulate), _ext.current_stream_ptr())
    _ext.check(rc)


def add_lora_bgmv(y: torch.Tensor, x: torch.Tensor, wa_T_all: torch.Tensor, wb_T_all: torch.Tensor,
                  indicies: torch.Tensor, layer_idx: int, scale: float) -> None:
    """Same arguments and in-place semantics as ``punica.ops.add_lora_bgmv`` at the reference's
    call sites (``lora_gpu.py:138,150,162``):
        y[i] += x[i] @ wa_T_all[indicies[i], layer_idx].T @ wb_T_all[indicies[i], layer_idx].T * scale
    with wa_T_all [N, L, r, Hin], wb_T_all [N, L, Hout, r], indicies int64 [B]."""
    _need_cuda(y, x, wa_T_all, wb_T_all, indicies)
    _need_contig(y, x, wa_T_all, wb_T_all, indicies)
    if indicies.dtype != torch.int64:
        raise TypeError("indicies must be int64 (as torch.randint produces at lora_gpu.py:120)")
    if wa_T_all.dim() != 4 or wb_T_all.dim() != 4:
        raise ValueError("wa_T_all must be [N, L, r, Hin] and wb_T_all [N, L, Hout, r]")
    N, L, r, hin = wa_T_all.shape
    N2, L2, hout, r2 = wb_T_all.shape
    if (N2, L2, r2) != (N, L, r):
        raise ValueError("wa_T_all and wb_T_all disagree on N, L or r")
    T = x.shape[0]
    if tuple(x.shape) != (T, hin) or tuple(y.shape) != (T, hout) or indicies.numel() != T:
        raise ValueError("x must be [B, Hin], y [B, Hout], indicies [B]")
    dt = _ext.dtype_code(x.dtype)
    if not (y.dtype == x.dtype == wa_T_all.dtype == wb_T_all.dtype):
        raise TypeError("y, x and the pool must share one 16-bit dtype")
    rc = _ext.lib().mlora_bgmv_reflayout(y.data_ptr(), x.data_ptr(), wa_T_all.data_ptr(), wb_T_all.data_ptr(),
                                         indicies.data_ptr(), T, N, L, r, hin, hout, layer_idx, float(scale), dt,
                                         _ext.current_stream_ptr())
    _ext.check(rc)


@dataclass
class RefDecodePlan:
    """Grouping of one decode batch by adapter for the reference-layout calls (written by ``mlora_reflayout_plan``)."""
    indicies: torch.Tensor         # int64 [T]
    group: int
    N: int
    L: int
    r: int
    buf: torch.Tensor              # uint8: perm, segments, chunks, counters, work records
    vws: Optional[torch.Tensor] = None

    @property
    def T(self) -> int:
        return self.indicies.numel()


def ref_rank_supported(r: int) -> bool:
    """Ranks the grouped reference-layout call takes (the plain ``add_lora_bgmv`` takes any rank up to 64)."""
    return r in (8, 16, 32, 64)


def plan_decode_ref(indicies: torch.Tensor, N: int, L: int, r: int, group: Optional[int] = None,
                    out: Optional[RefDecodePlan] = None) -> RefDecodePlan:
    """Group a decode batch by adapter for ``add_lora_bgmv_multi``: once per step, the plan serves every layer and
    projection that uses this index vector on pools of N adapters, L layers and rank r.  Pass `out` to reuse a
    plan's buffers (no allocation; safe under graph capture)."""
    _need_cuda(indicies)
    _need_contig(indicies)
    if indicies.dtype != torch.int64:
        raise TypeError("indicies must be int64 (as torch.randint produces at lora_gpu.py:120)")
    T = indicies.numel()
    if group is None:
        group = out.group if out is not None else min(4, default_group(T))
    lib = _ext.lib()
    if out is None:
        out = RefDecodePlan(indicies, group, N, L, r,
                            torch.empty(max(16, lib.mlora_reflayout_plan_bytes(T)), dtype=torch.uint8, device=indicies.device))
    else:
        if out.T != T or (out.N, out.L, out.r) != (N, L, r):
            raise ValueError("the plan to reuse was made for another batch size or pool")
        out.indicies, out.group = indicies, group
    _ext.check(lib.mlora_reflayout_plan(indicies.data_ptr(), T, N, L, r, group, out.buf.data_ptr(), out.buf.numel(),
                                        _ext.current_stream_ptr()))
    return out


def add_lora_bgmv_multi(ys: Sequence[torch.Tensor], xs: Sequence[torch.Tensor], was: Sequence[torch.Tensor],
                        wbs: Sequence[torch.Tensor], plan: RefDecodePlan, layer_idx: int, scale: float,
                        accumulate: bool = True) -> None:
    """``punica.ops.add_lora_bgmv`` for several projections of one layer in one call pair, on the reference's pool
    layout in place: ``ys[p][i] (+)= xs[p][i] @ was[p][idx[i], layer].T @ wbs[p][idx[i], layer].T * scale`` with
    was[p] [N, L, r, Hin], wbs[p] [N, L, Hout, r] and idx the index vector the plan was made from
    (``lora_gpu.py:137-138,149-150,161-162`` in one go).  ``accumulate=False`` defines ys as the delta alone
    (zeros for indices outside the pool), which saves the ``torch.zeros`` of ``lora_gpu.py:137``."""
    n = len(ys)
    if not (len(xs) == len(was) == len(wbs) == n) or not 1 <= n <= _ext.MAX_PROJ:
        raise ValueError(f"need 1..{_ext.MAX_PROJ} projections with one y, x, wa and wb each")
    _need_cuda(*ys, *xs, *was, *wbs)
    _need_contig(*ys, *xs, *was, *wbs)
    T = plan.T
    yv, xv, av, bv, hi, ho = _VoidArr(), _VoidArr(), _VoidArr(), _VoidArr(), _IntArr(), _IntArr()
    dt = ys[0].dtype
    for i in range(n):
        if was[i].dim() != 4 or wbs[i].dim() != 4:
            raise ValueError("wa_T_all must be [N, L, r, Hin] and wb_T_all [N, L, Hout, r]")
        N, L, r, hin = was[i].shape
        N2, L2, hout, r2 = wbs[i].shape
        if (N2, L2, r2) != (N, L, r) or (N, L, r) != (plan.N, plan.L, plan.r):
            raise ValueError("pool tensors disagree with each other or with the plan on N, L or r")
        if tuple(xs[i].shape) != (T, hin) or tuple(ys[i].shape) != (T, hout):
            raise ValueError("x must be [B, Hin] and y [B, Hout] for the plan's batch")
        if not (ys[i].dtype == xs[i].dtype == was[i].dtype == wbs[i].dtype == dt):
            raise TypeError("y, x and the pools must share one 16-bit dtype")
        yv[i], xv[i], av[i], bv[i], hi[i], ho[i] = ys[i].data_ptr(), xs[i].data_ptr(), was[i].data_ptr(), wbs[i].data_ptr(), hin, hout
    lib = _ext.lib()
    ws_bytes = lib.mlora_bgmv_workspace_bytes(n, T, max(hi[i] for i in range(n)), plan.r)
    if plan.vws is None or plan.vws.numel() < ws_bytes:
        plan.vws = torch.empty(ws_bytes, dtype=torch.uint8, device=ys[0].device)
    rc = lib.mlora_bgmv_reflayout_multi(n, yv, xv, av, bv, hi, ho, plan.buf.data_ptr(), T, plan.N, plan.L, plan.r, layer_idx,
                                        float(scale), plan.group, _ext.dtype_code(dt), int(accumulate),
                                        plan.vws.data_ptr(), plan.vws.numel(), _ext.current_stream_ptr())
    _ext.check(rc)


# ---------------------------------------------------------------------- prefill
def sgmv_workspace(T: int, n_seg: int, device, n_proj: int = 1) -> torch.Tensor:
    """Workspace for a prefill batch of T tokens in n_seg segments; n_proj > 1 sizes it for
    ``sgmv_multi`` calls of up to that many projections (it then also serves single ``sgmv`` calls)."""
    lib = _ext.lib()
    nbytes = max(lib.mlora_sgmv_workspace_bytes(T, n_seg), lib.mlora_sgmv_multi_workspace_bytes(T, n_seg, n_proj))
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


@dataclass
class PrefillPlan:
    """Tile list and per-tile records of one prefill batch, held in `workspace` (written by ``mlora_sgmv_plan``)."""
    seg_start: torch.Tensor
    seg_len: torch.Tensor
    seg_adapter: torch.Tensor
    T: int
    workspace: torch.Tensor


def _check_segments(seg_start, seg_len, seg_adapter):
    _need_cuda(seg_start, seg_len, seg_adapter)
    _need_contig(seg_start, seg_len, seg_adapter)
    for s in (seg_start, seg_len, seg_adapter):
        if s.dtype != torch.int32:
            raise TypeError("segment arrays must be int32")
    n_seg = seg_start.numel()
    if seg_len.numel() != n_seg or seg_adapter.numel() != n_seg:
        raise ValueError("seg_start, seg_len and seg_adapter must have the same length")
    return n_seg


def plan_prefill(seg_start: torch.Tensor, seg_len: torch.Tensor, seg_adapter: torch.Tensor, T: int,
                 pool: AdapterPool, workspace: Optional[torch.Tensor] = None, n_proj: int = 1,
                 aligned: bool = False) -> PrefillPlan:
    """Plan a prefill batch once; the plan serves every projection and layer (``sgmv(..., plan=plan)``,
    ``sgmv_multi(..., plan=plan)``, ``gemm_lora(..., plan)`` for up to `n_proj` projections per call).
    ``aligned`` cuts the tiles at multiples of 64 tokens (and at segment ends) rather than every 64 tokens of a
    segment: fewer tiles per 256-row block of ``gemm_lora``, a few more tiles overall."""
    n_seg = _check_segments(seg_start, seg_len, seg_adapter)
    if workspace is None:
        workspace = sgmv_workspace(T, n_seg, seg_start.device, n_proj)
    pool.sync()
    plan_fn = _ext.lib().mlora_sgmv_plan_aligned if aligned else _ext.lib().mlora_sgmv_plan
    rc = plan_fn(
        seg_start.data_ptr(), seg_len.data_ptr(), seg_adapter.data_ptr(), n_seg,
        _ext.ptr(pool.page_tbl), _ext.ptr(pool.rank), _ext.ptr(pool.scaling), T, pool.n_slots, pool.max_pages,
        pool.page_rows, pool.n_pages, pool.max_rank, workspace.data_ptr(), workspace.numel(), _ext.current_stream_ptr())
    _ext.check(rc)
    return PrefillPlan(seg_start, seg_len, seg_adapter, T, workspace)


def sgmv(y: torch.Tensor, x: torch.Tensor, pool: AdapterPool, layer: int, proj: str,
         seg_start: Optional[torch.Tensor] = None, seg_len: Optional[torch.Tensor] = None,
         seg_adapter: Optional[torch.Tensor] = None, accumulate: bool = True,
         workspace: Optional[torch.Tensor] = None, plan: Optional[PrefillPlan] = None) -> None:
    """Prefill LoRA apply over packed segments (one adapter per segment) on MFMA tiles.  Either pass the
    segment arrays (planned inside the call) or a `plan` from ``plan_prefill``."""
    if plan is not None:
        seg_start, seg_len, seg_adapter, workspace = plan.seg_start, plan.seg_len, plan.seg_adapter, plan.workspace
    _need_cuda(y, x)
    _need_contig(y, x)
    n_seg = _check_segments(seg_start, seg_len, seg_adapter)
    hin, hout = pool.projections[proj]
    T = x.shape[0]
    if plan is not None and plan.T != T:
        raise ValueError("plan was made for a different number of tokens")
    if tuple(x.shape) != (T, hin) or tuple(y.shape) != (T, hout):
        raise ValueError(f"expected x [{T}, {hin}] and y [{T}, {hout}]")
    if x.dtype != pool.dtype or y.dtype != pool.dtype:
        raise TypeError(f"x and y must have the pool dtype {pool.dtype}")
    if workspace is None:
        workspace = sgmv_workspace(T, n_seg, x.device)
    pool.sync()
    a_ptr, b_ptr = pool.slab_ptrs(layer, proj)
    fn = _ext.lib().mlora_sgmv_planned if plan is not None else _ext.lib().mlora_sgmv
    rc = fn(
        y.data_ptr(), x.data_ptr(), a_ptr, b_ptr, seg_start.data_ptr(), seg_len.data_ptr(), seg_adapter.data_ptr(),
        n_seg, _ext.ptr(pool.page_tbl), _ext.ptr(pool.rank), _ext.ptr(pool.scaling),
        T, hin, hout, pool.n_slots, pool.max_pages, pool.page_rows, pool.n_pages, pool.max_rank,
        pool.dtype_code, int(accumulate), workspace.data_ptr(), workspace.numel(), _ext.current_stream_ptr())
    _ext.check(rc)


def sgmv_multi(ys: Sequence[torch.Tensor], xs: Sequence[torch.Tensor], pool: AdapterPool, layer: int,
               projs: Sequence[str], plan: PrefillPlan, accumulate: bool = True) -> None:
    """Prefill LoRA apply for up to 8 projections of one layer against one plan, three launches in all.
    Projections listed next to each other with the same x tensor (q, k, v; gate, up) share its reads.
    The plan's workspace must have been sized for this many projections (``plan_prefill(..., n_proj=)``)."""
    n = len(projs)
    if not (len(ys) == len(xs) == n) or not 1 <= n <= _ext.MAX_PROJ:
        raise ValueError(f"need 1..{_ext.MAX_PROJ} projections with one y and one x each")
    _need_cuda(*ys, *xs)
    _need_contig(*ys, *xs)
    T = plan.T
    yv, xv, av, bv, hi, ho = _VoidArr(), _VoidArr(), _VoidArr(), _VoidArr(), _IntArr(), _IntArr()
    for i, p in enumerate(projs):
        hin, hout = pool.projections[p]
        if xs[i].dtype != pool.dtype or ys[i].dtype != pool.dtype:
            raise TypeError(f"x and y must have the pool dtype {pool.dtype}")
        if tuple(xs[i].shape) != (T, hin) or tuple(ys[i].shape) != (T, hout):
            raise ValueError(f"projection {p}: expected x [{T}, {hin}] and y [{T}, {hout}]")
        a_ptr, b_ptr = pool.slab_ptrs(layer, p)
        yv[i], xv[i], av[i], bv[i], hi[i], ho[i] = ys[i].data_ptr(), xs[i].data_ptr(), a_ptr, b_ptr, hin, hout
    n_seg = _check_segments(plan.seg_start, plan.seg_len, plan.seg_adapter)
    pool.sync()
    rc = _ext.lib().mlora_sgmv_multi_planned(
        n, yv, xv, av, bv, hi, ho, plan.seg_start.data_ptr(), plan.seg_len.data_ptr(), plan.seg_adapter.data_ptr(),
        n_seg, _ext.ptr(pool.page_tbl), _ext.ptr(pool.rank), _ext.ptr(pool.scaling), T, pool.n_slots, pool.max_pages,
        pool.page_rows, pool.n_pages, pool.max_rank, pool.dtype_code, int(accumulate),
        plan.workspace.data_ptr(), plan.workspace.numel(), _ext.current_stream_ptr())
    _ext.check(rc)


def gemm_lora(ys: Sequence[torch.Tensor], xs: Sequence[torch.Tensor], ws: Sequence[torch.Tensor], pool: Optional[AdapterPool],
              layer: int, projs: Sequence[str], plan: Optional[PrefillPlan]) -> None:
    """Base projection and LoRA in one pass for up to 8 projections of one prefill layer:
    ``ys[p] = xs[p] @ ws[p] + delta`` with ``ws[p]`` the base weight as ``[hin, hout]`` (the layout of
    ``layer_weight.q_weight_``), i.e. ``q = torch.mm(x, Wq); q += q_lora`` of
    ``transformer_layer_infer.py:145-147,160-171`` with q written once.  ``plan=None`` (then ``pool`` may be
    None and ``projs`` only names the outputs) runs the base products alone."""
    n = len(projs)
    if not (len(ys) == len(xs) == len(ws) == n) or not 1 <= n <= _ext.MAX_PROJ:
        raise ValueError(f"need 1..{_ext.MAX_PROJ} projections with one y, one x and one w each")
    _need_cuda(*ys, *xs, *ws)
    _need_contig(*ys, *xs, *ws)
    T = xs[0].shape[0]
    if plan is not None and plan.T != T:
        raise ValueError("plan was built for a different number of tokens")
    yv, xv, wv, av, bv, hi, ho = _VoidArr(), _VoidArr(), _VoidArr(), _VoidArr(), _VoidArr(), _IntArr(), _IntArr()
    dtype = xs[0].dtype
    for i, p in enumerate(projs):
        hin, hout = ws[i].shape
        if plan is not None and tuple(pool.projections[p]) != (hin, hout):
            raise ValueError(f"projection {p}: base weight is {tuple(ws[i].shape)}, the pool has {pool.projections[p]}")
        if not (xs[i].dtype == ys[i].dtype == ws[i].dtype == dtype) or (plan is not None and dtype != pool.dtype):
            raise TypeError("x, y, w and the pool must share one 16-bit dtype")
        if tuple(xs[i].shape) != (T, hin) or tuple(ys[i].shape) != (T, hout):
            raise ValueError(f"projection {p}: expected x [{T}, {hin}] and y [{T}, {hout}]")
        yv[i], xv[i], wv[i], hi[i], ho[i] = ys[i].data_ptr(), xs[i].data_ptr(), ws[i].data_ptr(), hin, hout
        if plan is not None:
            av[i], bv[i] = pool.slab_ptrs(layer, p)
    if plan is None:
        rc = _ext.lib().mlora_gemm_lora_planned(n, yv, xv, wv, None, None, hi, ho, None, None, None, 0, None, None, None, T,
                                                0, 0, 0, 0, 16, _ext.dtype_code(dtype), None, 0, _ext.current_stream_ptr())
    else:
        n_seg = _check_segments(plan.seg_start, plan.seg_len, plan.seg_adapter)
        pool.sync()
        rc = _ext.lib().mlora_gemm_lora_planned(
            n, yv, xv, wv, av, bv, hi, ho, plan.seg_start.data_ptr(), plan.seg_len.data_ptr(), plan.seg_adapter.data_ptr(),
            n_seg, _ext.ptr(pool.page_tbl), _ext.ptr(pool.rank), _ext.ptr(pool.scaling), T, pool.n_slots, pool.max_pages,
            pool.page_rows, pool.n_pages, pool.max_rank, pool.dtype_code,
            plan.workspace.data_ptr(), plan.workspace.numel(), _ext.current_stream_ptr())
    _ext.check(rc)


def lora_prefill_ref(x: torch.Tensor, A_T: torch.Tensor, B_T: torch.Tensor, layer_idx: int,
                     workspace: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The reference's prefill expression on its own layout (``lora_gpu.py:125-128``):
    ``torch.bmm(torch.bmm(x, A_T[:bsz, layer].transpose(-1,-2)), B_T[:bsz, layer].transpose(-1,-2))``
    with x [bsz, Lpad, Hin], A_T [>=bsz, L, r, Hin], B_T [>=bsz, L, Hout, r]; request b uses slot b."""
    _need_cuda(x, A_T, B_T)
    _need_contig(x, A_T, B_T)
    bsz, lpad, hin = x.shape
    n, L, r, hin2 = A_T.shape
    _, _, hout, _ = B_T.shape
    if hin2 != hin or n < bsz or B_T.shape[0] < bsz or B_T.shape[1] != L or B_T.shape[3] != r:
        raise ValueError("x, A_T and B_T shapes do not fit the reference prefill call")
    if not (x.dtype == A_T.dtype == B_T.dtype):
        raise TypeError("x and the pool must share one 16-bit dtype")
    if out is None:
        y = torch.empty((bsz, lpad, hout), dtype=x.dtype, device=x.device)
    else:
        y = out
        if tuple(y.shape) != (bsz, lpad, hout) or y.dtype != x.dtype or not y.is_contiguous() or not y.is_cuda:
            raise ValueError("out must be a contiguous device tensor [bsz, Lpad, Hout] of x's dtype")
    if workspace is None:
        workspace = sgmv_workspace(bsz * lpad, bsz, x.device)
    rc = _ext.lib().mlora_prefill_reflayout(y.data_ptr(), x.data_ptr(), A_T.data_ptr(), B_T.data_ptr(), bsz, lpad, L, r,
                                            hin, hout, layer_idx, _ext.dtype_code(x.dtype), workspace.data_ptr(),
                                            workspace.numel(), _ext.current_stream_ptr())
    _ext.check(rc)
    return y


# ---------------------------------------------------------------------- one-call surface
def lora_apply(y: torch.Tensor, x: torch.Tensor, tok_adapter: torch.Tensor, pool: AdapterPool, layer: int,
               proj: str, plan: Optional[DecodePlan] = None) -> torch.Tensor:
    """y (the base projection output, [T, Hout]) += LoRA delta of every token's adapter; returns y."""
    bgmv([y], [x], pool, layer, [proj], tok_adapter, plan=plan, accumulate=True)
    return y
