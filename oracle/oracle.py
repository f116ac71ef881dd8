"""ctypes front end of the CPU checker (``mlora_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()``
and by ``bench.py``'s cpu_baseline leg, never by the shipped package.  All
arrays are numpy; 16-bit floats travel as ``uint16`` bit patterns
(``np.float16.view(np.uint16)`` for fp16, the upper half of the fp32 pattern
for bf16) so fp16 and bf16 share one code path.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmlora_oracle.so")
_lib = None

FP16, BF16 = 0, 1


def build(force: bool = False) -> str:
    """Compile the checker with gcc (a few hundred ms)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_f16_to_f32.restype = C.c_float
        _lib.orc_f16_to_f32.argtypes = [C.c_uint16]
        _lib.orc_f32_to_f16.restype = C.c_uint16
        _lib.orc_f32_to_f16.argtypes = [C.c_float]
    return _lib


def _p(a, ct=None):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be contiguous"
    return a.ctypes.data_as(C.c_void_p)


def _check(rc, what):
    if rc == -2:
        raise IndexError(f"{what}: adapter index or rank out of range")
    if rc != 0:
        raise ValueError(f"{what}: invalid argument (rc={rc})")


# ---------------------------------------------------------------- conversions
def to_bits(a: np.ndarray, dtype: int) -> np.ndarray:
    """fp32 array -> uint16 bit patterns of the 16-bit type (round to nearest even)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, np.uint16)
    fn = lib().orc_f32_to_f16_n if dtype == FP16 else lib().orc_f32_to_bf16_n
    fn(_p(a), _p(out), C.c_size_t(a.size))
    return out


def from_bits(b: np.ndarray, dtype: int) -> np.ndarray:
    b = np.ascontiguousarray(b, dtype=np.uint16)
    out = np.empty(b.shape, np.float32)
    fn = lib().orc_f16_to_f32_n if dtype == FP16 else lib().orc_bf16_to_f32_n
    fn(_p(b), _p(out), C.c_size_t(b.size))
    return out


# ---------------------------------------------------------------- index work
def pool_gather(tok_adapter, page_tbl, rank, scaling, page_rows):
    tok_adapter = np.ascontiguousarray(tok_adapter, np.int32)
    page_tbl = np.ascontiguousarray(page_tbl, np.int32)
    rank = np.ascontiguousarray(rank, np.int32)
    scaling = np.ascontiguousarray(scaling, np.float32)
    T = tok_adapter.size
    N, max_pages = page_tbl.shape
    row_off = np.empty((T, max_pages), np.int32)
    out_rank = np.empty(T, np.int32)
    out_scale = np.empty(T, np.float32)
    rc = lib().orc_pool_gather(_p(tok_adapter), T, _p(page_tbl), _p(rank), _p(scaling), N, max_pages,
                               page_rows, _p(row_off), _p(out_rank), _p(out_scale))
    _check(rc, "pool_gather")
    return row_off, out_rank, out_scale


def pool_scatter(src, dst_slab, pages, page_rows):
    """In place: rows of `src` [rank, W] onto the pages `pages` of `dst_slab` [n_pages * page_rows, W]."""
    src = np.ascontiguousarray(src)
    assert dst_slab.flags["C_CONTIGUOUS"] and dst_slab.dtype == src.dtype and dst_slab.shape[1] == src.shape[1]
    pages = np.ascontiguousarray(pages, np.int32)
    fn = lib().orc_pool_scatter
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int64]
    rc = fn(_p(src), _p(dst_slab), src.shape[1] * src.itemsize, _p(pages), pages.size, src.shape[0], page_rows,
            dst_slab.shape[0] // page_rows)
    _check(rc, "pool_scatter")
    return dst_slab


def build_segments(tok_adapter, n_adapters):
    tok_adapter = np.ascontiguousarray(tok_adapter, np.int32)
    T = tok_adapter.size
    cap = max(1, min(T, n_adapters))
    perm = np.empty(T, np.int32)
    seg_start = np.zeros(cap, np.int32)
    seg_len = np.zeros(cap, np.int32)
    seg_adapter = np.zeros(cap, np.int32)
    n_seg = C.c_int32(0)
    n_valid = C.c_int32(0)
    rc = lib().orc_build_segments(_p(tok_adapter), T, n_adapters, _p(perm), _p(seg_start), _p(seg_len),
                                  _p(seg_adapter), C.byref(n_seg), C.byref(n_valid))
    _check(rc, "build_segments")
    n = n_seg.value
    return perm, seg_start[:n].copy(), seg_len[:n].copy(), seg_adapter[:n].copy(), n_valid.value


def build_chunks(seg_start, seg_len, seg_adapter, n_valid, T, group):
    seg_start = np.ascontiguousarray(seg_start, np.int32)
    seg_len = np.ascontiguousarray(seg_len, np.int32)
    seg_adapter = np.ascontiguousarray(seg_adapter, np.int32)
    cap = max(1, T)
    cs = np.zeros(cap, np.int32)
    cl = np.zeros(cap, np.int32)
    ca = np.zeros(cap, np.int32)
    nc = C.c_int32(0)
    rc = lib().orc_build_chunks(_p(seg_start), _p(seg_len), _p(seg_adapter), seg_start.size, n_valid, T,
                                group, _p(cs), _p(cl), _p(ca), C.byref(nc))
    _check(rc, "build_chunks")
    n = nc.value
    return cs[:n].copy(), cl[:n].copy(), ca[:n].copy()


WORK_WORDS = 80


def work_cap(T):
    return ((T + 7) // 8) * 8


def build_work(chunk_start, chunk_len, chunk_adapter, perm, page_tbl, rank, scaling, page_rows, n_pages, T):
    cs = np.ascontiguousarray(chunk_start, np.int32)
    cl = np.ascontiguousarray(chunk_len, np.int32)
    ca = np.ascontiguousarray(chunk_adapter, np.int32)
    perm = np.ascontiguousarray(perm, np.int32)
    page_tbl = np.ascontiguousarray(page_tbl, np.int32)
    rank = np.ascontiguousarray(rank, np.int32)
    scaling = np.ascontiguousarray(scaling, np.float32)
    cap = work_cap(T)
    work = np.empty((cap, WORK_WORDS), np.int32)
    rc = lib().orc_build_work(_p(cs), _p(cl), _p(ca), cs.size, _p(perm), _p(page_tbl), _p(rank), _p(scaling),
                              page_tbl.shape[1], page_rows, C.c_int64(n_pages), cap, _p(work))
    _check(rc, "build_work")
    return work


def sgmv_plan(seg_start, seg_len, tile, aligned=False):
    seg_start = np.ascontiguousarray(seg_start, np.int32)
    seg_len = np.ascontiguousarray(seg_len, np.int32)
    cap = int(sum((int(l) + tile - 1) // tile + 1 for l in seg_len)) + 1
    ts = np.zeros(cap, np.int32)
    t0 = np.zeros(cap, np.int32)
    tn = np.zeros(cap, np.int32)
    n = C.c_int32(0)
    fn = lib().orc_sgmv_plan_aligned if aligned else lib().orc_sgmv_plan
    rc = fn(_p(seg_start), _p(seg_len), seg_start.size, tile, _p(ts), _p(t0), _p(tn), C.byref(n))
    _check(rc, "sgmv_plan")
    return ts[:n.value].copy(), t0[:n.value].copy(), tn[:n.value].copy()


# ---------------------------------------------------------------- arithmetic
def lora_apply_paged(x, a_rows, b_rows, tok_adapter, a_page_tbl, b_page_tbl, rank, scaling,
                     page_rows, dtype, y0=None, acc64=False):
    """y = round16(y0 + s_a (x A_a) B_a) over the paged pool; all 16-bit arrays as uint16 bits."""
    x = np.ascontiguousarray(x, np.uint16)
    a_rows = np.ascontiguousarray(a_rows, np.uint16)
    b_rows = np.ascontiguousarray(b_rows, np.uint16)
    tok_adapter = np.ascontiguousarray(tok_adapter, np.int32)
    a_page_tbl = np.ascontiguousarray(a_page_tbl, np.int32)
    b_page_tbl = np.ascontiguousarray(b_page_tbl, np.int32)
    rank = np.ascontiguousarray(rank, np.int32)
    scaling = np.ascontiguousarray(scaling, np.float32)
    T, Hin = x.shape
    Hout = b_rows.shape[1]
    assert a_rows.shape[1] == Hin
    N, max_pages = a_page_tbl.shape
    if y0 is not None:
        y0 = np.ascontiguousarray(y0, np.uint16)
        assert y0.shape == (T, Hout)
    y = np.empty((T, Hout), np.uint16)
    rc = lib().orc_lora_apply_paged(_p(y), _p(y0), _p(x), _p(a_rows), _p(b_rows), _p(tok_adapter),
                                    _p(a_page_tbl), _p(b_page_tbl), _p(rank), _p(scaling),
                                    T, Hin, Hout, N, max_pages, page_rows, dtype, int(acc64))
    _check(rc, "lora_apply_paged")
    return y


def gemm_lora_paged(x, w, a_rows, b_rows, tok_adapter, a_page_tbl, b_page_tbl, rank, scaling, page_rows, dtype,
                    acc64=False, ref_rounding=False):
    """y = round16(x W + s_a (x A_a) B_a) (or the reference's three roundings); 16-bit arrays as uint16 bits."""
    x = np.ascontiguousarray(x, np.uint16)
    w = np.ascontiguousarray(w, np.uint16)
    a_rows = np.ascontiguousarray(a_rows, np.uint16)
    b_rows = np.ascontiguousarray(b_rows, np.uint16)
    tok_adapter = np.ascontiguousarray(tok_adapter, np.int32)
    a_page_tbl = np.ascontiguousarray(a_page_tbl, np.int32)
    b_page_tbl = np.ascontiguousarray(b_page_tbl, np.int32)
    rank = np.ascontiguousarray(rank, np.int32)
    scaling = np.ascontiguousarray(scaling, np.float32)
    T, Hin = x.shape
    Hout = w.shape[1]
    assert w.shape[0] == Hin and a_rows.shape[1] == Hin and b_rows.shape[1] == Hout
    N, max_pages = a_page_tbl.shape
    y = np.empty((T, Hout), np.uint16)
    rc = lib().orc_gemm_lora_paged(_p(y), _p(x), _p(w), _p(a_rows), _p(b_rows), _p(tok_adapter), _p(a_page_tbl),
                                   _p(b_page_tbl), _p(rank), _p(scaling), T, Hin, Hout, N, max_pages, page_rows,
                                   dtype, int(acc64), int(ref_rounding))
    _check(rc, "gemm_lora_paged")
    return y


def add_lora_bgmv_ref(y, x, wa_T_all, wb_T_all, indices, layer_idx, scale, dtype=FP16):
    """In place y += scale * x @ wa[idx, layer].T @ wb[idx, layer].T on the reference layout."""
    assert y.dtype == np.uint16 and y.flags["C_CONTIGUOUS"]
    x = np.ascontiguousarray(x, np.uint16)
    wa = np.ascontiguousarray(wa_T_all, np.uint16)
    wb = np.ascontiguousarray(wb_T_all, np.uint16)
    idx = np.ascontiguousarray(indices, np.int64)
    N, L, r, Hin = wa.shape
    Hout = wb.shape[2]
    assert wb.shape == (N, L, Hout, r)
    T = x.shape[0]
    rc = lib().orc_add_lora_bgmv_ref(_p(y), _p(x), _p(wa), _p(wb), _p(idx), T, N, L, r, Hin, Hout,
                                     layer_idx, C.c_float(scale), dtype)
    _check(rc, "add_lora_bgmv_ref")
    return y


def prefill_bmm_ref(x, A_T, B_T, layer_idx, dtype=FP16, round_mid=False):
    x = np.ascontiguousarray(x, np.uint16)
    A_T = np.ascontiguousarray(A_T, np.uint16)
    B_T = np.ascontiguousarray(B_T, np.uint16)
    Bsz, Lpad, Hin = x.shape
    _, L, r, _ = A_T.shape
    Hout = B_T.shape[2]
    y = np.empty((Bsz, Lpad, Hout), np.uint16)
    rc = lib().orc_prefill_bmm_ref(_p(y), _p(x), _p(A_T), _p(B_T), Bsz, Lpad, L, r, Hin, Hout, layer_idx,
                                   dtype, int(round_mid))
    _check(rc, "prefill_bmm_ref")
    return y


def cpu_lora_worker(x, down, up):
    x = np.ascontiguousarray(x, np.uint16)
    down = np.ascontiguousarray(down, np.float32)
    up = np.ascontiguousarray(up, np.float32)
    n, Hin = x.shape
    r, Hout = up.shape
    out = np.empty((n, Hout), np.uint16)
    rc = lib().orc_cpu_lora_worker(_p(x), _p(down), _p(up), _p(out), n, Hin, Hout, r)
    _check(rc, "cpu_lora_worker")
    return out


def cpu_chunk_plan(batch, tkn_num, cap):
    cpr = (tkn_num - 1) // cap + 1
    req = np.zeros(batch * cpr, np.int32)
    tok0 = np.zeros(batch * cpr, np.int32)
    ntok = np.zeros(batch * cpr, np.int32)
    n = C.c_int32(0)
    rc = lib().orc_cpu_chunk_plan(batch, tkn_num, cap, _p(req), _p(tok0), _p(ntok), C.byref(n))
    _check(rc, "cpu_chunk_plan")
    return req[:n.value], tok0[:n.value], ntok[:n.value]


def cpu_lora_batch(x, down, up, req_adapter, tkn_num, cap, n_threads=1):
    """Delta for a batch of equal-length requests, sharded (request, chunk) over n_threads."""
    x = np.ascontiguousarray(x, np.uint16)
    down = np.ascontiguousarray(down, np.float32)
    up = np.ascontiguousarray(up, np.float32)
    req_adapter = np.ascontiguousarray(req_adapter, np.int32)
    batch = req_adapter.size
    _, Hin, r = down.shape
    Hout = up.shape[2]
    assert x.shape == (batch * tkn_num, Hin)
    out = np.empty((batch * tkn_num, Hout), np.uint16)
    rc = lib().orc_cpu_lora_batch(_p(x), _p(down), _p(up), _p(out), _p(req_adapter), batch, tkn_num, cap,
                                  Hin, Hout, r, n_threads)
    _check(rc, "cpu_lora_batch")
    return out


class CpuLoraPool:
    """Persistent worker threads for ``cpu_lora_batch`` (created once, woken per batch): the way the
    reference runs its CPU workers, so that thread creation is not part of a timed batch."""

    def __init__(self, n_threads: int):
        fn = lib().orc_cpu_pool_create
        fn.restype = C.c_void_p
        fn.argtypes = [C.c_int]
        self._h = fn(n_threads)
        if not self._h:
            raise ValueError("cannot create a CPU worker pool with that many threads")
        self.n_threads = n_threads

    def run(self, x, down, up, req_adapter, tkn_num, cap, out=None):
        x = np.ascontiguousarray(x, np.uint16)
        down = np.ascontiguousarray(down, np.float32)
        up = np.ascontiguousarray(up, np.float32)
        req_adapter = np.ascontiguousarray(req_adapter, np.int32)
        batch = req_adapter.size
        _, Hin, r = down.shape
        Hout = up.shape[2]
        assert x.shape == (batch * tkn_num, Hin)
        if out is None:
            out = np.empty((batch * tkn_num, Hout), np.uint16)
        fn = lib().orc_cpu_pool_run
        fn.argtypes = [C.c_void_p] * 6 + [C.c_int] * 6
        rc = fn(self._h, _p(x), _p(down), _p(up), _p(out), _p(req_adapter), batch, tkn_num, cap, Hin, Hout, r)
        _check(rc, "cpu_pool_run")
        return out

    def close(self):
        if self._h:
            fn = lib().orc_cpu_pool_destroy
            fn.argtypes = [C.c_void_p]
            fn.restype = None
            fn(self._h)
            self._h = None

    def __del__(self):
        self.close()
