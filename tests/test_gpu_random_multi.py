"""GPU parity on drawn shapes: the multi-projection calls (decode `bgmv` over up to 7 projections, prefill
`sgmv_multi` and `gemm_lora` over the same) with the number of projections, their widths, which of them share an
input, ranks, dtype, batch and launch form drawn from a seed, every projection against the oracle
(`orc.lora_apply_paged` / `orc.gemm_lora_paged`, rtol 1e-2 / atol 1e-3).  The fixed cases elsewhere pin the
benchmark's shapes; these pin the index arithmetic in between (projection and slice numbering, shared-input groups,
column blocks, many-round launches) on shapes nobody chose.
"""
import numpy as np
import pytest
import torch

from gpu_common import assert_close_bits, oracle_apply, say, tdtype, upload_pool
from helpers import BF16, FP16, PagedPool, bits_of, bits_to_torch, torch_to_bits
from mlora import bgmv, gemm_lora, plan_decode, plan_prefill, sgmv_multi
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def _draw_pool(rng, wmax):
    n = int(rng.integers(1, 30))
    ranks = [rng.integers(1, 17, n), rng.integers(1, 33, n), rng.integers(1, 65, n), rng.choice([8, 16, 32, 64], n)][int(rng.integers(0, 4))]
    n_proj = int(rng.integers(1, 8))
    dtype = FP16 if rng.integers(0, 2) else BF16
    shapes, xid = [], []
    for p in range(n_proj):
        if p > 0 and rng.random() < 0.5:
            hin = shapes[-1][0]
            xid.append(xid[-1])                                # reads the previous projection's input tensor
        else:
            hin = int(rng.integers(1, wmax)) * 8
            xid.append(p)
        shapes.append((hin, int(rng.integers(1, wmax)) * 8))
    names = [f"p{i}" for i in range(n_proj)]
    pps = []
    for hin, hout in shapes:
        pp = PagedPool(np.random.default_rng(12345), ranks, hin, hout, page_rows=8, dtype=dtype)    # one page table for all
        r2 = np.random.default_rng(rng.integers(1 << 30))
        pp.a_rows = bits_of((r2.standard_normal(pp.a_rows.shape) * 0.02).astype(np.float32), dtype)
        pp.b_rows = bits_of((r2.standard_normal(pp.b_rows.shape) * 0.02).astype(np.float32), dtype)
        pps.append(pp)
    pool = upload_pool(pps[0], projections=dict(zip(names, shapes)))
    for nm, pp in zip(names, pps):
        pool.a_rows[nm][0].copy_(bits_to_torch(pp.a_rows, dtype))
        pool.b_rows[nm][0].copy_(bits_to_torch(pp.b_rows, dtype))
    return n, ranks, names, shapes, xid, dtype, pps, pool


def _draw_inputs(rng, T, shapes, xid, dtype):
    xs = {}
    for p, (hin, _) in enumerate(shapes):
        if xid[p] not in xs:
            xs[xid[p]] = bits_of(rng.standard_normal((T, hin)).astype(np.float32), dtype)
    y0 = [bits_of(rng.standard_normal((T, hout)).astype(np.float32), dtype) for _, hout in shapes]
    return xs, y0


def _outputs(y0, acc, dtype):
    return [bits_to_torch(y, dtype, "cuda") if acc else torch.full(y.shape, float("nan"), dtype=tdtype(dtype), device="cuda")
            for y in y0]


# seeds 2, 5 and 6 draw batches of 1500-3333 tokens (launches of many rounds), the others 1-700
@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 7, 8])
def test_decode_multi_projection_drawn(seed):
    rng = np.random.default_rng(7000 + seed)
    big = seed in (2, 5, 6)
    n, ranks, names, shapes, xid, dtype, pps, pool = _draw_pool(rng, 130 if big else 400)
    T = int(rng.choice([1500, 2048, 2500, 3333]) if big else rng.choice([1, 5, 64, 100, 257, 512, 700]))
    tok = rng.integers(-1, n + 1, T).astype(np.int32)          # -1 and n name no adapter
    if rng.random() < 0.3:
        p = np.arange(1, n + 1, dtype=np.float64) ** -1.2
        tok = rng.choice(n, T, p=p / p.sum()).astype(np.int32)
    group = int(rng.choice([1, 2, 4, 8]))
    if group == 8 and ranks.max() > 32:
        group = 4
    fused = [False, None, True][int(rng.integers(0, 3))]
    acc = bool(rng.integers(0, 2))
    xs, y0 = _draw_inputs(rng, T, shapes, xid, dtype)
    say(f"decode drawn seed={seed} n={n} rmax={ranks.max()} shapes={shapes} xid={xid} dt={dtype} T={T} group={group} "
        f"fused={fused} acc={acc}")
    xt = {k: bits_to_torch(v, dtype, "cuda") for k, v in xs.items()}
    ys = _outputs(y0, acc, dtype)
    t = torch.from_numpy(tok).cuda()
    bgmv(ys, [xt[xid[p]] for p in range(len(names))], pool, 0, names, t, plan=plan_decode(t, pool, group=group),
         accumulate=acc, fused=fused)
    torch.cuda.synchronize()
    tok_o = np.where((tok >= 0) & (tok < n), tok, -1).astype(np.int32)
    for p in range(len(names)):
        want = oracle_apply(pps[p], xs[xid[p]], tok_o, y0[p] if acc else None)
        assert_close_bits(torch_to_bits(ys[p]), want, dtype, f"seed {seed} projection {p}")


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_prefill_multi_projection_drawn(seed):
    rng = np.random.default_rng(8000 + seed)
    n, ranks, names, shapes, xid, dtype, pps, pool = _draw_pool(rng, 400)
    k = int(rng.integers(1, 12))
    lens = rng.choice([1, 5, 63, 64, 65, 127, 128, 129, 200, 30, 500], k).astype(np.int32)
    gaps = (rng.integers(0, 4, k) * (rng.random(k) < 0.3)).astype(np.int32)
    ad = rng.integers(-1, n, k).astype(np.int32)
    start, pos = [], 0
    for l, g in zip(lens, gaps):
        pos += int(g)
        start.append(pos)
        pos += int(l)
    T = pos + int(rng.integers(0, 3))
    tok = np.full(T, -1, np.int32)
    for s, l, a in zip(start, lens, ad):
        tok[s:s + l] = a
    acc, aligned = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    xs, y0 = _draw_inputs(rng, T, shapes, xid, dtype)
    say(f"prefill drawn seed={seed} n={n} rmax={ranks.max()} shapes={shapes} xid={xid} dt={dtype} T={T} segs={k} "
        f"acc={acc} aligned={aligned}")
    xt = {kk: bits_to_torch(v, dtype, "cuda") for kk, v in xs.items()}
    ys = _outputs(y0, acc, dtype)
    d = [torch.from_numpy(np.asarray(a, np.int32)).cuda() for a in (start, lens, ad)]
    plan = plan_prefill(d[0], d[1], d[2], T, pool, n_proj=len(names), aligned=aligned)
    x_list = [xt[xid[p]] for p in range(len(names))]
    sgmv_multi(ys, x_list, pool, 0, names, plan, accumulate=acc)
    ws = [bits_of((rng.standard_normal(s) / np.sqrt(s[0])).astype(np.float32), dtype) for s in shapes]
    yg = _outputs(y0, False, dtype)
    gemm_lora(yg, x_list, [bits_to_torch(w, dtype, "cuda") for w in ws], pool, 0, names, plan)
    torch.cuda.synchronize()
    for p in range(len(names)):
        want = oracle_apply(pps[p], xs[xid[p]], tok, y0[p] if acc else None)
        assert_close_bits(torch_to_bits(ys[p]), want, dtype, f"seed {seed} sgmv projection {p}")
        pp = pps[p]
        want_g = orc.gemm_lora_paged(xs[xid[p]], ws[p], pp.a_rows, pp.b_rows, tok, pp.page_tbl, pp.page_tbl, pp.ranks,
                                     pp.scaling, pp.page_rows, pp.dtype)
        assert_close_bits(torch_to_bits(yg[p]), want_g, dtype, f"seed {seed} gemm_lora projection {p}")
