"""Helpers shared by the GPU parity tests: upload a numpy paged pool, run, compare with the oracle."""
from __future__ import annotations

import sys

import numpy as np
import torch

from helpers import BF16, FP16, PagedPool, bits_to_torch, f32_of, torch_to_bits
from mlora import AdapterPool
from oracle import oracle as orc

RTOL, ATOL = 1e-2, 1e-3     # the tolerance the build's contract states for fp16 and bf16


def say(msg):
    """Name the case before it touches the GPU (flushed, so a lost box still shows it)."""
    print(f"[gpu-case] {msg}", flush=True)
    sys.stdout.flush()


def tdtype(dtype):
    return torch.float16 if dtype == FP16 else torch.bfloat16


def upload_pool(pp: PagedPool, projections=None, n_layers=1):
    """AdapterPool on the GPU holding exactly the numpy pool's rows and tables (projection 'p')."""
    projections = projections or {"p": (pp.hin, pp.hout)}
    pool = AdapterPool(n_layers, projections, pp.n, pp.n_pages, page_rows=pp.page_rows,
                       max_rank=max(1, pp.max_pages * pp.page_rows if pp.max_pages * pp.page_rows <= 64 else 64),
                       dtype=tdtype(pp.dtype), device="cuda")
    assert pool.max_pages == pp.max_pages, (pool.max_pages, pp.max_pages)
    pool.h_page_tbl[:] = pp.page_tbl
    pool.h_rank[:] = pp.ranks
    pool.h_scaling[:] = pp.scaling
    pool._dirty = True
    pool.sync()
    if "p" in projections:
        pool.a_rows["p"][0].copy_(bits_to_torch(pp.a_rows, pp.dtype))
        pool.b_rows["p"][0].copy_(bits_to_torch(pp.b_rows, pp.dtype))
    return pool


def oracle_apply(pp: PagedPool, x_bits, tok, y0_bits=None, acc64=False):
    return orc.lora_apply_paged(x_bits, pp.a_rows, pp.b_rows, tok, pp.page_tbl, pp.page_tbl, pp.ranks, pp.scaling,
                                pp.page_rows, pp.dtype, y0=y0_bits, acc64=acc64)


def assert_close_bits(got_bits, want_bits, dtype, what=""):
    got = f32_of(got_bits, dtype).astype(np.float64)
    want = f32_of(want_bits, dtype).astype(np.float64)
    err = np.abs(got - want)
    tol = ATOL + RTOL * np.abs(want)
    bad = err > tol
    assert not bad.any(), (f"{what}: {int(bad.sum())} of {bad.size} elements outside rtol {RTOL} / atol {ATOL}; "
                           f"worst |err| {err.max():.3e} at {np.unravel_index(err.argmax(), err.shape)}")
    return float(err.max())
