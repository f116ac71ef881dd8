"""Config 4 in the forms the benchmark times: the prefill batch of `bench.py --workload c4` (seed 1004: 16 requests
of U[128, 1024] tokens, each on one of 32 rank-64 adapters, bf16, Llama-13B widths 5120 / 13824) through
`sgmv_multi` over the seven projections q, k, v, o, gate, up, down in one call (shared-x shrink groups of three,
K splits in proportion to K, expand blocks of 640 / 576 columns), and the same batch with base weights through
`gemm_lora` (`bench.py --workload f1`).  Replaces the three `torch.bmm` pairs of lora_gpu.py:127-128,145-146,157-158.

Every token of every projection is checked against an fp32 evaluation on the device; sampled tokens of the first and
the last segment (and the tokens either side of every segment boundary) against the CPU oracle.  A second, small
batch with 127 / 128 / 129-token segments, a gap and an adapter-less segment goes through the same seven
projections in accumulate and in delta mode and is checked against the oracle in full.  Tolerance rtol 1e-2 / atol 1e-3.
"""
import numpy as np
import pytest
import torch

import bench
from gpu_common import ATOL, RTOL, say
from mlora import _ext, gemm_lora, plan_prefill, sgmv_multi, sgmv_workspace, workloads
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

RANK = 64


def _oracle_rows(pool, p, adapters):
    """Rows of the given adapters copied into a small dense pool for the CPU oracle."""
    pages_per = RANK // pool.page_rows
    a_rows = torch.cat([pool.a_rows[p][0][pool.rows_of(int(a))] for a in adapters]).view(torch.int16).cpu().numpy().view(np.uint16)
    b_rows = torch.cat([pool.b_rows[p][0][pool.rows_of(int(a))] for a in adapters]).view(torch.int16).cpu().numpy().view(np.uint16)
    tbl = np.arange(len(adapters) * pages_per, dtype=np.int32).reshape(len(adapters), pages_per)
    return a_rows, b_rows, tbl


def _bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def _check_sample_against_oracle(pool, p, x, y0, got, tok_adapter, sample, w=None):
    ads = np.unique(tok_adapter[sample])
    ads = ads[ads >= 0]
    remap = {int(a): i for i, a in enumerate(ads)}
    a_rows, b_rows, tbl = _oracle_rows(pool, p, ads)
    tok = np.array([remap.get(int(tok_adapter[t]), -1) for t in sample], np.int32)
    idx = torch.from_numpy(np.asarray(sample)).cuda()
    rank = np.full(len(ads), RANK, np.int32)
    scaling = pool.h_scaling[ads].astype(np.float32)
    if w is None:
        want = orc.lora_apply_paged(_bits(x[idx]), a_rows, b_rows, tok, tbl, tbl, rank, scaling, pool.page_rows, orc.BF16,
                                    y0=None if y0 is None else _bits(y0[idx]))
    else:
        want = orc.gemm_lora_paged(_bits(x[idx]), _bits(w), a_rows, b_rows, tok, tbl, tbl, rank, scaling, pool.page_rows, orc.BF16)
    want = orc.from_bits(want, orc.BF16)
    have = got[idx].float().cpu().numpy()
    err = np.abs(have - want)
    assert np.all(err <= ATOL + RTOL * np.abs(want)), (p, float(err.max()))


def _device_delta(pool, p, x, tok_adapter):
    """fp32 on the device: s_a (x A_a^T) B_a for the tokens of every adapter, zero elsewhere."""
    hout = pool.b_rows[p].shape[-1]
    d = torch.zeros(x.shape[0], hout, device=x.device, dtype=torch.float32)
    for a in np.unique(tok_adapter[tok_adapter >= 0]):
        idx = torch.from_numpy(np.nonzero(tok_adapter == a)[0]).cuda()
        rows = pool.rows_of(int(a))
        A = pool.a_rows[p][0][rows].float()
        B = pool.b_rows[p][0][rows].float()
        d[idx] = float(pool.h_scaling[a]) * ((x[idx].float() @ A.t()) @ B)
    return d


def _expect_block_widths(T, n_seg, names, projections):
    lib = _ext.lib()
    cols = {p: lib.mlora_sgmv_expand_cols(T, n_seg, len(names), projections[p][1]) for p in names}
    # the widths whose block count per tile suits the tile-major order: the paths this file is about
    assert all(cols[p] == (640 if projections[p][1] == 5120 else 576) for p in names), cols


def test_config4_batch_as_the_benchmark_times_it():
    dev = torch.device("cuda:0")
    b = bench._c4_batch(dev, True)
    T, projections, pool, names, x_in, w = b["T"], b["projections"], b["pool"], b["names"], b["x_in"], b["w"]
    starts, lens, adapters = (t.cpu().numpy() for t in b["seg"])
    assert names == ["q", "k", "v", "o", "gate", "up", "down"] and len(lens) == 16 and T == int(lens.sum())
    _expect_block_widths(T, 16, names, projections)
    tok_adapter = np.repeat(adapters, lens).astype(np.int32)
    rng = np.random.default_rng(404)
    first = np.arange(starts[0], starts[0] + lens[0])
    last = np.arange(starts[-1], starts[-1] + lens[-1])
    edges = np.unique(np.clip(np.concatenate([starts - 1, starts, starts + lens - 1]), 0, T - 1))
    sample = np.unique(np.concatenate([rng.choice(first, 12, replace=False), rng.choice(last, 12, replace=False),
                                       [first[0], first[-1], last[0], last[-1]], edges]))

    # --- sgmv_multi, accumulate (the bench's c4 step)
    y0 = {p: b["y"][p].clone() for p in names}
    y = {p: b["y"][p] for p in names}
    say(f"config 4: sgmv_multi over 7 projections, T={T}, 16 segments, bf16, rank 64")
    plan = plan_prefill(*b["seg"], T, pool, workspace=b["ws"])
    sgmv_multi([y[p] for p in names], [x_in[p] for p in names], pool, 0, names, plan)
    torch.cuda.synchronize()
    for p in names:
        want = y0[p].float() + _device_delta(pool, p, x_in[p], tok_adapter)
        err = (y[p].float() - want).abs()
        assert bool((err <= ATOL + RTOL * want.abs()).all()), (p, float(err.max()))
        _check_sample_against_oracle(pool, p, x_in[p], y0[p], y[p], tok_adapter, sample)
        del want, err

    # --- gemm_lora over the same seven (the bench's f1 step)
    yg = {p: torch.full((T, projections[p][1]), float("nan"), device=dev, dtype=torch.bfloat16) for p in names}
    say(f"config 4: gemm_lora over 7 projections, T={T}")
    gplan = plan_prefill(*b["seg"], T, pool, workspace=b["ws"], aligned=True)
    gemm_lora([yg[p] for p in names], [x_in[p] for p in names], [w[p] for p in names], pool, 0, names, gplan)
    torch.cuda.synchronize()
    for p in names:
        want = x_in[p].float() @ w[p].float() + _device_delta(pool, p, x_in[p], tok_adapter)
        err = (yg[p].float() - want).abs()
        assert bool((err <= ATOL + RTOL * want.abs()).all()), (p, float(err.max()))
        del want, err
        _check_sample_against_oracle(pool, p, x_in[p], None, yg[p], tok_adapter, sample[:: max(1, len(sample) // 24)], w=w[p])


@pytest.mark.parametrize("accumulate", [True, False], ids=["accumulate", "delta"])
def test_config4_widths_small_batch_against_the_oracle(accumulate):
    """127 / 128 / 129-token segments, a gap, an adapter-less segment and a tail at Llama-13B widths: all seven
    projections in one call, every element against the oracle."""
    dev = torch.device("cuda:0")
    projections = workloads.LLAMA13B_ALL
    names = list(projections)
    rng = np.random.default_rng(1404)
    pool_ranks = np.full(6, RANK, np.int32)
    from mlora import AdapterPool
    pool = AdapterPool(1, projections, 6, 6 * 8 + 5, page_rows=8, max_rank=RANK, dtype=torch.bfloat16, device=dev)
    workloads.fill_pool(pool, pool_ranks, np.array([0.5, 1.0, 0.25, 2.0, 0.5, 1.0], np.float32), rng, seed=1404)
    lens = np.array([127, 128, 129, 40, 64], np.int32)
    gaps = np.array([0, 0, 3, 0, 0], np.int32)
    starts = (np.cumsum(lens + gaps) - lens).astype(np.int32)
    adapters = np.array([4, 0, 5, -1, 2], np.int32)
    T = int(starts[-1] + lens[-1]) + 7
    tok_adapter = np.full(T, -1, np.int32)
    for s, l, a in zip(starts, lens, adapters):
        tok_adapter[s:s + l] = a
    _expect_block_widths(T, len(lens), names, projections)
    gen = torch.Generator(device=dev).manual_seed(14)
    xs = {h: torch.randn(T, h, device=dev, generator=gen).bfloat16() for h in (5120, 13824)}
    x_ffn = torch.randn(T, 5120, device=dev, generator=gen).bfloat16()
    x_in = {"q": xs[5120], "k": xs[5120], "v": xs[5120], "o": x_ffn, "gate": x_ffn, "up": x_ffn, "down": xs[13824]}
    y0 = {p: torch.randn(T, projections[p][1], device=dev, generator=gen).bfloat16() for p in names}
    y = {p: (y0[p].clone() if accumulate else torch.full_like(y0[p], float("nan"))) for p in names}
    seg = tuple(torch.from_numpy(a).to(dev) for a in (starts, lens, adapters))
    ws = sgmv_workspace(T, len(lens), dev, n_proj=len(names))
    plan = plan_prefill(*seg, T, pool, workspace=ws)
    say(f"config-4 widths, small batch T={T}, accumulate={accumulate}")
    sgmv_multi([y[p] for p in names], [x_in[p] for p in names], pool, 0, names, plan, accumulate=accumulate)
    torch.cuda.synchronize()
    used = np.unique(adapters[adapters >= 0])
    remap = np.full(6, -1, np.int32)
    remap[used] = np.arange(len(used))
    tok = np.where(tok_adapter >= 0, remap[np.maximum(tok_adapter, 0)], -1).astype(np.int32)
    for p in names:
        a_rows, b_rows, tbl = _oracle_rows(pool, p, used)
        want = orc.lora_apply_paged(_bits(x_in[p]), a_rows, b_rows, tok, tbl, tbl, np.full(len(used), RANK, np.int32),
                                    pool.h_scaling[used].astype(np.float32), pool.page_rows, orc.BF16,
                                    y0=_bits(y0[p]) if accumulate else None)
        want = orc.from_bits(want, orc.BF16)
        have = y[p].float().cpu().numpy()
        if accumulate:
            outside = tok_adapter < 0
            assert np.array_equal(_bits(y[p])[outside], _bits(y0[p])[outside]), p     # untouched, bit for bit
        err = np.abs(have - want)
        assert np.all(err <= ATOL + RTOL * np.abs(want)), (p, float(err.max()))

    # the same batch through gemm_lora (base weights of modest size are drawn per projection)
    if accumulate:
        w = {p: (torch.randn(projections[p], device=dev, generator=gen) / projections[p][0] ** 0.5).bfloat16() for p in names}
        yg = {p: torch.full((T, projections[p][1]), float("nan"), device=dev, dtype=torch.bfloat16) for p in names}
        gplan = plan_prefill(*seg, T, pool, workspace=ws, aligned=True)
        say(f"config-4 widths, small batch T={T}, gemm_lora")
        gemm_lora([yg[p] for p in names], [x_in[p] for p in names], [w[p] for p in names], pool, 0, names, gplan)
        torch.cuda.synchronize()
        for p in names:
            a_rows, b_rows, tbl = _oracle_rows(pool, p, used)
            sub = np.concatenate([np.arange(0, T, 29), [126, 127, 128, 254, 255, 256, 257, T - 1]])
            idx = torch.from_numpy(sub).cuda()
            want = orc.gemm_lora_paged(_bits(x_in[p][idx]), _bits(w[p]), a_rows, b_rows, tok[sub], tbl, tbl,
                                       np.full(len(used), RANK, np.int32), pool.h_scaling[used].astype(np.float32),
                                       pool.page_rows, orc.BF16)
            want = orc.from_bits(want, orc.BF16)
            have = yg[p][idx].float().cpu().numpy()
            err = np.abs(have - want)
            assert np.all(err <= ATOL + RTOL * np.abs(want)), (p, float(err.max()))
