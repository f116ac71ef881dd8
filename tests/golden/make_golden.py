#!/usr/bin/env python3
"""Writes tests/golden/*.npz: small seeded inputs with the outputs the CPU checker (oracle/) gives
for them.  The reference ships no vectors for this path, so these are this build's own known-answer
files; they freeze the checker's behaviour (a later change to oracle/ that alters a result fails
tests/test_golden.py) and give the GPU tests fixed data.  Run from the repository root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [ROOT, os.path.join(ROOT, "tests")]

from helpers import BF16, FP16, PagedPool, bits_of  # noqa: E402
from oracle import oracle as orc  # noqa: E402


def apply_case(seed, dtype, ranks, hin, hout, T, page_rows):
    rng = np.random.default_rng(seed)
    pp = PagedPool(rng, ranks, hin, hout, page_rows=page_rows, dtype=dtype)
    tok = rng.integers(-1, len(ranks), T).astype(np.int32)
    x = bits_of(rng.standard_normal((T, hin)).astype(np.float32), dtype)
    y0 = bits_of(rng.standard_normal((T, hout)).astype(np.float32), dtype)
    args = (x, pp.a_rows, pp.b_rows, tok, pp.page_tbl, pp.page_tbl, pp.ranks, pp.scaling, page_rows, dtype)
    return dict(dtype=dtype, page_rows=page_rows, a_rows=pp.a_rows, b_rows=pp.b_rows, page_tbl=pp.page_tbl,
                rank=pp.ranks, scaling=pp.scaling, tok=tok, x=x, y0=y0,
                y_acc=orc.lora_apply_paged(*args, y0=y0), y_delta=orc.lora_apply_paged(*args, y0=None))


def gather_case(seed, T, N, group, page_rows):
    rng = np.random.default_rng(seed)
    rank = rng.choice([8, 16, 32, 64], N).astype(np.int32)
    mp = -(-64 // page_rows)
    page_tbl = np.full((N, mp), -1, np.int32)
    nxt = 0
    for i, r in enumerate(rank):
        k = -(-int(r) // page_rows)
        page_tbl[i, :k] = np.arange(nxt, nxt + k)
        nxt += k
    page_tbl = page_tbl[:, :]                    # contiguous page ids; the kernel only copies them
    scaling = (32.0 / rank).astype(np.float32)
    p = np.arange(1, N + 1, dtype=np.float64) ** -1.0
    tok = rng.choice(N, size=T, p=p / p.sum()).astype(np.int32)
    tok[rng.random(T) < 0.05] = -1
    perm, ss, sl, sa, nv = orc.build_segments(tok, N)
    cs, cl, ca = orc.build_chunks(ss, sl, sa, nv, T, group)
    ro, rk, sc = orc.pool_gather(tok, page_tbl, rank, scaling, page_rows)
    work = orc.build_work(cs, cl, ca, perm, page_tbl, rank, scaling, page_rows, nxt, T)
    return dict(work=work, tok=tok, page_tbl=page_tbl, rank=rank, scaling=scaling, page_rows=page_rows, group=group, n_pages=nxt,
                perm=perm, seg_start=ss, seg_len=sl, seg_adapter=sa, n_valid=nv, chunk_start=cs, chunk_len=cl,
                chunk_adapter=ca, row_off=ro, tok_rank=rk, tok_scale=sc)


def ref_case(seed):
    rng = np.random.default_rng(seed)
    N, L, r, hin, hout, T, layer = 6, 3, 16, 256, 384, 11, 2
    wa = bits_of((rng.standard_normal((N, L, r, hin)) * 0.05).astype(np.float32), FP16)
    wb = bits_of((rng.standard_normal((N, L, hout, r)) * 0.05).astype(np.float32), FP16)
    idx = rng.integers(0, N, T).astype(np.int64)
    x = bits_of(rng.standard_normal((T, hin)).astype(np.float32), FP16)
    y0 = bits_of(rng.standard_normal((T, hout)).astype(np.float32), FP16)
    y = y0.copy()
    orc.add_lora_bgmv_ref(y, x, wa, wb, idx, layer, 1.0)
    xp = bits_of(rng.standard_normal((3, 20, hin)).astype(np.float32), FP16)
    yp = orc.prefill_bmm_ref(xp, wa[:3], wb[:3], layer, FP16, round_mid=False)
    return dict(wa=wa, wb=wb, idx=idx, x=x, y0=y0, y=y, layer=layer, xp=xp, yp=yp)


def main():
    np.savez_compressed(os.path.join(HERE, "apply_fp16.npz"), **apply_case(11, FP16, [8, 16, 32, 64, 5], 256, 192, 23, 8))
    np.savez_compressed(os.path.join(HERE, "apply_bf16.npz"), **apply_case(12, BF16, [16, 16, 64, 24], 512, 128, 17, 8))
    np.savez_compressed(os.path.join(HERE, "gather.npz"), **gather_case(13, 300, 40, 4, 8))
    np.savez_compressed(os.path.join(HERE, "reflayout.npz"), **ref_case(14))


if __name__ == "__main__":
    main()
