"""ctypes binding of ``libmlora_cpu.so`` (C ABI declared in ``include/mlora_cpu.h``): the CPU side of the
CPU-assisted LoRA path -- the worker arithmetic of ``lora_cpu/lora_shm_op/app.py:136-141`` on a persistent
thread pool, and the in-process workers of the transport (``app.py:102-143``).

Host code only: nothing here touches the GPU, and there is no fallback if the library has not been built.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmlora_cpu.so")
CSRC_DIR = os.path.normpath(os.path.join(_HERE, "..", "csrc", "cpu"))

OK, EINVAL, ERANGE, ESTATE = 0, -1, -2, -3
W_F32, W_F16 = 0, 1
MAX_RANK, MAX_THREADS, ASSIST_MAX_PROJ = 256, 1024, 4

_vp, _i32, _i64, _f32 = C.c_void_p, C.c_int, C.c_int64, C.c_float

# name -> (restype, argtypes); one entry per function declared in include/mlora_cpu.h
SIGNATURES = {
    "mlora_cpu_last_error": (C.c_char_p, []),
    "mlora_cpu_version": (_i32, []),
    "mlora_cpu_pool_create": (_vp, [_i32]),
    "mlora_cpu_pool_destroy": (None, [_vp]),
    "mlora_cpu_pool_threads": (_i32, [_vp]),
    "mlora_cpu_lora": (_i32, [_vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _f32, _i32]),
    "mlora_cpu_assist_start": (_vp, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _i32, _i32,
                                     _i32, _vp, _i32, _i32]),
    "mlora_cpu_assist_stop": (_i32, [_vp, _vp, _vp]),
}

_lib = None


class MloraCpuError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"mlora_cpu error {code}: {message}")
        self.code = code


def lib() -> C.CDLL:
    """Load the library (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}`")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def _check(rc: int) -> None:
    if rc != OK:
        raise MloraCpuError(rc, lib().mlora_cpu_last_error().decode("utf-8", "replace"))


def _weights(a, what: str):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float32:
        return a, W_F32
    if a.dtype in (np.float16, np.uint16):
        return a, W_F16
    raise TypeError(f"{what} must be float32 or binary16 (float16 / uint16 bit patterns), got {a.dtype}")


def _u16(a, what: str):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    if a.dtype != np.uint16:
        raise TypeError(f"{what} must be binary16 (float16 / uint16 bit patterns), got {a.dtype}")
    return a


class CpuLoraPool:
    """Persistent worker threads (created once, woken per batch), as the reference keeps its CPU LoRA workers
    alive between batches (``runServerCPULoRA.py:74-90``)."""

    def __init__(self, n_threads: int):
        self._h = lib().mlora_cpu_pool_create(int(n_threads))
        if not self._h:
            raise MloraCpuError(ERANGE, lib().mlora_cpu_last_error().decode("utf-8", "replace"))
        self.n_threads = lib().mlora_cpu_pool_threads(self._h)

    @property
    def handle(self):
        if not self._h:
            raise MloraCpuError(ESTATE, "the pool has been closed")
        return self._h

    def close(self) -> None:
        if self._h:
            lib().mlora_cpu_pool_destroy(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        self.close()


def cpu_lora(x, A, B, tok_adapter, y0=None, out=None, scale: float = 1.0, tokens_per_task: int = 8,
             pool: Optional[CpuLoraPool] = None) -> np.ndarray:
    """``out[t] = half(y0[t] + scale * (x[t].float() @ A[a] @ B[a]))`` with ``a = tok_adapter[t]`` on the host
    cores; x ``[T, Hin]`` binary16, A ``[N, Hin, r]``, B ``[N, r, Hout]`` fp32 or binary16.  Returns uint16 bit
    patterns ``[T, Hout]``.  ``pool=None`` runs on the calling thread."""
    x = _u16(x, "x")
    A, wa = _weights(A, "A")
    B, wb = _weights(B, "B")
    if wa != wb:
        raise TypeError("A and B must have the same dtype")
    tok = np.ascontiguousarray(tok_adapter, np.int32)
    if A.ndim != 3 or B.ndim != 3 or x.ndim != 2:
        raise ValueError("x must be [T, Hin], A [N, Hin, r], B [N, r, Hout]")
    N, Hin, r = A.shape
    N2, r2, Hout = B.shape
    T = x.shape[0]
    if (N2, r2) != (N, r) or x.shape[1] != Hin or tok.shape != (T,):
        raise ValueError("shapes of x, A, B and tok_adapter do not fit")
    if y0 is not None:
        y0 = _u16(y0, "y0")
        if y0.shape != (T, Hout):
            raise ValueError("y0 must be [T, Hout]")
    if out is None:
        out = np.empty((T, Hout), np.uint16)
    elif out.dtype != np.uint16 or out.shape != (T, Hout) or not out.flags.c_contiguous:
        raise ValueError("out must be a contiguous uint16 array [T, Hout]")
    rc = lib().mlora_cpu_lora(pool.handle if pool is not None else None, x.ctypes.data, A.ctypes.data, B.ctypes.data, wa,
                              tok.ctypes.data, y0.ctypes.data if y0 is not None else None, out.ctypes.data,
                              T, Hin, Hout, r, N, float(scale), int(tokens_per_task))
    _check(rc)
    return out


class AssistWorkers:
    """In-process workers of the CPU-assist transport: a polling thread over the signal table that hands every
    woken (request chunk, projection) to the pool and clears the signal when the rows are written
    (``app.py:102-143``; one thread pool instead of one pinned process per chunk and projection).

    ``x_slots`` / ``out_slots[q]`` are ``[n_slots, slot_tokens, H]`` uint16 arrays, ``signals`` int16
    ``[n_proj, n_workers]``, ``tkn_len`` int32 ``[1]`` -- host views of the transport's buffers;
    ``down[q]`` ``[N, H, r]`` and ``up[q]`` ``[N, r, H]`` the adapters of projection q, ``slot_adapter`` int32
    ``[n_slots]`` the adapter of the request in each slot (None: adapter 0).  The arrays must outlive the object."""

    def __init__(self, pool: CpuLoraPool, x_slots: np.ndarray, out_slots: Sequence[np.ndarray], signals: np.ndarray,
                 tkn_len: np.ndarray, cap: int, down: Sequence[np.ndarray], up: Sequence[np.ndarray],
                 slot_adapter: Optional[np.ndarray] = None, sig_base: int = 2, sig_stride: int = 200):
        n_proj = len(out_slots)
        if not (len(down) == len(up) == n_proj) or not 1 <= n_proj <= ASSIST_MAX_PROJ:
            raise ValueError(f"need 1..{ASSIST_MAX_PROJ} projections with one out_slots, down and up each")
        if x_slots.dtype != np.uint16 or x_slots.ndim != 3 or not x_slots.flags.c_contiguous:
            raise ValueError("x_slots must be a contiguous uint16 array [n_slots, slot_tokens, H]")
        n_slots, slot_tokens, H = x_slots.shape
        if signals.dtype != np.int16 or signals.ndim != 2 or signals.shape[0] != n_proj or not signals.flags.c_contiguous:
            raise ValueError("signals must be a contiguous int16 array [n_proj, n_workers]")
        if tkn_len.dtype != np.int32 or tkn_len.size < 1:
            raise ValueError("tkn_len must be an int32 array")
        self._keep = [pool, x_slots, signals, tkn_len]
        dn, upw, wd = [], [], None
        for q in range(n_proj):
            o = out_slots[q]
            if o.dtype != np.uint16 or o.shape != x_slots.shape or not o.flags.c_contiguous:
                raise ValueError("every out_slots[q] must match x_slots")
            d, w1 = _weights(down[q], "down")
            u, w2 = _weights(up[q], "up")
            if w1 != w2 or (wd is not None and w1 != wd):
                raise TypeError("all weights must share one dtype")
            wd = w1
            if d.ndim != 3 or u.ndim != 3 or d.shape[1] != H or u.shape[2] != H or d.shape[0] != u.shape[0] or d.shape[2] != u.shape[1]:
                raise ValueError("down[q] must be [N, H, r] and up[q] [N, r, H]")
            dn.append(d)
            upw.append(u)
            self._keep += [o, d, u]
        N, _, r = dn[0].shape
        if any(d.shape != dn[0].shape for d in dn):
            raise ValueError("all projections must have the same adapter count and rank")
        sa = None
        if slot_adapter is not None:
            sa = np.ascontiguousarray(slot_adapter, np.int32)
            if sa.shape != (n_slots,):
                raise ValueError("slot_adapter must be [n_slots]")
            self._keep.append(sa)
        VP = C.c_void_p * n_proj
        self._h = lib().mlora_cpu_assist_start(
            pool.handle, x_slots.ctypes.data, VP(*[o.ctypes.data for o in out_slots]), signals.ctypes.data,
            tkn_len.ctypes.data, n_proj, signals.shape[1], n_slots, slot_tokens, H, int(cap),
            VP(*[d.ctypes.data for d in dn]), VP(*[u.ctypes.data for u in upw]), wd, r, N,
            sa.ctypes.data if sa is not None else None, sig_base, sig_stride)
        if not self._h:
            raise MloraCpuError(EINVAL, lib().mlora_cpu_last_error().decode("utf-8", "replace"))
        self.served = self.rejected = 0

    def stop(self):
        """End the polling thread once the chunks in flight are done; returns (served, rejected)."""
        if self._h:
            s, r = C.c_int64(0), C.c_int64(0)
            rc = lib().mlora_cpu_assist_stop(self._h, C.byref(s), C.byref(r))
            self._h = None
            _check(rc)
            self.served, self.rejected = s.value, r.value
            self._keep = []
        return self.served, self.rejected

    def __del__(self):
        self.stop()
