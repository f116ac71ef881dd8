"""Randomised parity sweep: small random shapes (token counts, adapter counts, ranks, widths with ragged
tails, adapter-less tokens, gaps between segments) through every decode form and the prefill forms,
each against the oracle.  Seeds are fixed; a failure names its seed."""
import numpy as np
import pytest
import torch

from gpu_common import assert_close_bits, oracle_apply, say, upload_pool
from helpers import BF16, FP16, PagedPool, bits_of, bits_to_torch, torch_to_bits
from mlora import bgmv, plan_decode, plan_prefill, sgmv, sgmv_multi

pytestmark = pytest.mark.gpu


def _widths(rng):
    return int(rng.choice([8, 72, 200, 512, 1032, 2056, 4096])), int(rng.choice([8, 72, 264, 512, 1024, 2064, 4104]))


@pytest.mark.parametrize("seed", range(16))
def test_random_decode(seed):
    rng = np.random.default_rng(1000 + seed)
    dtype = FP16 if seed % 2 else BF16
    N = int(rng.integers(1, 40))
    ranks = rng.choice([1, 3, 8, 16, 24, 32, 48, 64], N)
    if seed % 4 == 0:
        ranks = np.minimum(ranks, 16)                       # rank-16 kernels
    elif seed % 4 == 1:
        ranks = np.minimum(ranks, 32)
    hin, hout = _widths(rng)
    T = int(rng.choice([1, 2, 7, 33, 64, 100, 257]))
    pp = PagedPool(rng, ranks, hin, hout, page_rows=int(rng.choice([4, 8, 16])), dtype=dtype)
    pool = upload_pool(pp)
    tok = rng.integers(-1, N, T).astype(np.int32)
    x = bits_of(rng.standard_normal((T, hin)).astype(np.float32), dtype)
    y0 = bits_of(rng.standard_normal((T, hout)).astype(np.float32), dtype)
    want = oracle_apply(pp, x, tok, y0)
    want_d = oracle_apply(pp, x, tok, None)
    t = torch.from_numpy(tok).cuda()
    xt = bits_to_torch(x, dtype, "cuda")
    groups = [1, 2, 4] + ([8] if pool.max_rank <= 32 else [])
    for group in [0] + groups:
        for fused in ([True] if group == 0 else [True, False]):
            for acc in (True, False):
                y = bits_to_torch(y0, dtype, "cuda") if acc else torch.full((T, hout), float("nan"), device="cuda", dtype=xt.dtype)
                say(f"random decode seed={seed} T={T} N={N} {hin}x{hout} max_rank={pool.max_rank} group={group} fused={fused} acc={acc}")
                bgmv([y], [xt], pool, 0, ["p"], t, plan=plan_decode(t, pool, group=group) if group else None,
                     accumulate=acc, fused=fused)
                torch.cuda.synchronize()
                assert_close_bits(torch_to_bits(y), want if acc else want_d, dtype, f"seed {seed} group {group} fused {fused}")


@pytest.mark.parametrize("seed", range(10))
def test_random_prefill(seed):
    rng = np.random.default_rng(2000 + seed)
    dtype = BF16 if seed % 2 else FP16
    N = int(rng.integers(1, 12))
    ranks = rng.choice([2, 8, 16, 24, 32, 64], N)
    if seed % 3 == 0:
        ranks = np.minimum(ranks, 16)
    hin, hout = _widths(rng)
    n_seg = int(rng.integers(1, 7))
    lens = rng.choice([0, 1, 5, 63, 64, 65, 130], n_seg)
    gaps = rng.choice([0, 0, 3], n_seg)
    starts = np.cumsum(np.r_[gaps[0], lens[:-1] + gaps[1:]]).astype(np.int32)
    T = int(starts[-1] + lens[-1] + rng.choice([0, 2]))
    if T == 0:
        T, lens[0] = 4, 4
    adapters = rng.integers(-1, N, n_seg).astype(np.int32)
    tok = np.full(T, -1, np.int32)
    for s, l, a in zip(starts, lens, adapters):
        tok[s:s + l] = a
    pp = PagedPool(rng, ranks, hin, hout, page_rows=8, dtype=dtype)
    pool = upload_pool(pp)
    x = bits_of(rng.standard_normal((T, hin)).astype(np.float32), dtype)
    y0 = bits_of(rng.standard_normal((T, hout)).astype(np.float32), dtype)
    want = oracle_apply(pp, x, tok, y0)
    d = [torch.from_numpy(np.asarray(a, np.int32)).cuda() for a in (starts, lens, adapters)]
    xt = bits_to_torch(x, dtype, "cuda")
    say(f"random prefill seed={seed} T={T} segs={n_seg} {hin}x{hout} max_rank={pool.max_rank}")
    y1 = bits_to_torch(y0, dtype, "cuda")
    sgmv(y1, xt, pool, 0, "p", d[0], d[1], d[2])
    plan = plan_prefill(d[0], d[1], d[2], T, pool, n_proj=2)
    y2, y3 = bits_to_torch(y0, dtype, "cuda"), bits_to_torch(y0, dtype, "cuda")
    sgmv_multi([y2, y3], [xt, xt], pool, 0, ["p", "p"], plan)       # the same projection twice: both must agree
    torch.cuda.synchronize()
    assert_close_bits(torch_to_bits(y1), want, dtype, f"seed {seed} sgmv")
    assert_close_bits(torch_to_bits(y2), want, dtype, f"seed {seed} sgmv_multi")
    assert torch.equal(y2, y3)
    covered = tok >= 0
    assert np.array_equal(torch_to_bits(y2)[~covered], y0[~covered])


@pytest.mark.parametrize("seed", range(12))
def test_random_gemm_lora(seed):
    """Base projection + LoRA in one pass on random shapes: few and many K steps with and without a partial one,
    ragged row and column tiles, empty and tiny segments, gaps, adapter-less segments, both tile cuts."""
    from mlora import gemm_lora
    from oracle import oracle as orc
    rng = np.random.default_rng(3000 + seed)
    dtype = BF16 if seed % 2 else FP16
    N = int(rng.integers(1, 9))
    ranks = rng.choice([1, 4, 8, 16, 24, 32, 48, 64], N)
    if seed % 3 == 0:
        ranks = np.minimum(ranks, 16)
    elif seed % 3 == 1:
        ranks = np.minimum(ranks, 32)
    hin = int(rng.choice([8, 40, 64, 96, 136, 256, 328, 520]))
    hout = int(rng.choice([8, 72, 256, 264, 520]))
    n_seg = int(rng.integers(1, 9))
    lens = rng.choice([0, 1, 5, 63, 64, 65, 130, 257], n_seg)
    gaps = rng.choice([0, 0, 3], n_seg)
    starts = np.cumsum(np.r_[gaps[0], lens[:-1] + gaps[1:]]).astype(np.int32)
    T = int(starts[-1] + lens[-1] + rng.choice([0, 2]))
    if T == 0:
        T, lens[0] = 4, 4
    adapters = rng.integers(-1, N, n_seg).astype(np.int32)
    tok = np.full(T, -1, np.int32)
    for s, l, a in zip(starts, lens, adapters):
        tok[s:s + l] = a
    pp = PagedPool(rng, ranks, hin, hout, page_rows=8, dtype=dtype)
    pool = upload_pool(pp)
    x = bits_of(rng.standard_normal((T, hin)).astype(np.float32), dtype)
    w = bits_of((rng.standard_normal((hin, hout)) / np.sqrt(hin)).astype(np.float32), dtype)
    want = orc.gemm_lora_paged(x, w, pp.a_rows, pp.b_rows, tok, pp.page_tbl, pp.page_tbl, pp.ranks, pp.scaling,
                               pp.page_rows, dtype)
    d = [torch.from_numpy(np.asarray(a, np.int32)).cuda() for a in (starts, lens, adapters)]
    xt, wt = bits_to_torch(x, dtype, "cuda"), bits_to_torch(w, dtype, "cuda")
    for aligned in (False, True):
        say(f"random gemm_lora seed={seed} T={T} segs={n_seg} {hin}x{hout} max_rank={pool.max_rank} aligned={aligned}")
        y = torch.full((T, hout), float("nan"), dtype=xt.dtype, device="cuda")
        gemm_lora([y], [xt], [wt], pool, 0, ["p"], plan_prefill(d[0], d[1], d[2], T, pool, aligned=aligned))
        torch.cuda.synchronize()
        assert_close_bits(torch_to_bits(y), want, dtype, f"seed {seed} aligned {aligned}")
