"""GPU parity: adapter-pool index/offset gather and grouping, bit-exact against the oracle."""
import numpy as np
import pytest
import torch

from gpu_common import say
from mlora import AdapterPool, _ext, plan_decode
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def _pool(n, ranks, page_rows, rng):
    need = [-(-int(r) // page_rows) for r in ranks]
    pool = AdapterPool(1, {"p": (64, 64)}, n, sum(need) + 2, page_rows=page_rows, max_rank=64, device="cuda")
    order = rng.permutation(pool.n_pages)
    pos = 0
    for i, (r, k) in enumerate(zip(ranks, need)):
        pool.allocate(i, int(r), 32.0 / r, pages=[int(p) for p in order[pos:pos + k]])
        pos += k
    pool.sync()
    return pool


def _check(tok, pool, group, n_bad_expected=0):
    T = len(tok)
    t = torch.from_numpy(tok).cuda()
    plan = plan_decode(t, pool, group=group, per_token=True)
    torch.cuda.synchronize()
    cnt = plan.counters.cpu().numpy()
    clean = np.where(tok >= pool.n_slots, -1, tok).astype(np.int32)      # bad ids count as "no adapter"
    perm, ss, sl, sa, nv = orc.build_segments(clean, pool.n_slots)
    cs, cl, ca = orc.build_chunks(ss, sl, sa, nv, T, group)
    ro, rk, sc = orc.pool_gather(clean, pool.h_page_tbl, pool.h_rank, pool.h_scaling, pool.page_rows)
    assert cnt[_ext.CNT_NSEG] == len(ss) and cnt[_ext.CNT_NVALID] == nv
    assert cnt[_ext.CNT_NCHUNK] == len(cs) and cnt[_ext.CNT_BAD] == n_bad_expected
    assert np.array_equal(plan.perm.cpu().numpy()[:T], perm)
    n = len(ss)
    assert np.array_equal(plan.seg_start.cpu().numpy()[:n], ss)
    assert np.array_equal(plan.seg_len.cpu().numpy()[:n], sl)
    assert np.array_equal(plan.seg_adapter.cpu().numpy()[:n], sa)
    n = len(cs)
    assert np.array_equal(plan.chunk_start.cpu().numpy()[:n], cs)
    assert np.array_equal(plan.chunk_len.cpu().numpy()[:n], cl)
    assert np.array_equal(plan.chunk_adapter.cpu().numpy()[:n], ca)
    want_work = orc.build_work(cs, cl, ca, perm, pool.h_page_tbl, pool.h_rank, pool.h_scaling, pool.page_rows,
                               pool.n_pages, T)
    assert np.array_equal(plan.work.cpu().numpy()[:want_work.shape[0]], want_work)
    assert np.array_equal(plan.row_off.cpu().numpy()[:T], ro)
    assert np.array_equal(plan.tok_rank.cpu().numpy()[:T], rk)
    assert np.array_equal(plan.tok_scale.cpu().numpy()[:T].view(np.uint32), sc.view(np.uint32))


@pytest.mark.parametrize("T,N,group,page_rows", [
    (1, 1, 1, 8), (2, 3, 2, 8), (7, 4, 4, 1), (64, 8, 8, 8), (256, 64, 4, 8), (512, 1000, 4, 8), (1000, 17, 2, 16),
    (1024, 128, 8, 8), (1025, 128, 1, 8), (4096, 300, 4, 8), (8192, 64, 4, 8), (8191, 5000, 8, 4)])
def test_gather_random(T, N, group, page_rows):
    rng = np.random.default_rng(T * 7 + N)
    ranks = rng.choice([8, 16, 32, 64], N)
    pool = _pool(N, ranks, page_rows, rng)
    p = np.arange(1, N + 1, dtype=np.float64) ** -1.1
    tok = rng.choice(N, size=T, p=p / p.sum()).astype(np.int32)
    say(f"gather zipf T={T} N={N} group={group} page_rows={page_rows}")
    _check(tok, pool, group)
    tok2 = rng.integers(-1, N, T).astype(np.int32)
    say(f"gather uniform+none T={T} N={N} group={group}")
    _check(tok2, pool, group)


def test_gather_edge_cases():
    rng = np.random.default_rng(99)
    pool = _pool(6, [8, 64, 16, 32, 8, 24], 8, rng)
    say("gather all tokens one adapter")
    _check(np.full(300, 3, np.int32), pool, 4)
    say("gather no token has an adapter")
    _check(np.full(77, -1, np.int32), pool, 8)
    say("gather every token its own adapter")
    _check(np.arange(6, dtype=np.int32)[::-1].copy(), pool, 2)
    tok = np.array([0, 6, 2, 100, -1, 5, 5, 2 ** 30], np.int32)      # three ids outside the pool
    say("gather with out-of-range adapter ids")
    _check(tok, pool, 4, n_bad_expected=3)


def test_gather_reuses_buffers_and_is_idempotent():
    rng = np.random.default_rng(5)
    pool = _pool(16, rng.choice([8, 16], 16), 8, rng)
    tok = torch.from_numpy(rng.integers(0, 16, 200).astype(np.int32)).cuda()
    say("gather twice into the same plan")
    plan = plan_decode(tok, pool, group=4)
    torch.cuda.synchronize()
    n = int(plan.counters[_ext.CNT_NCHUNK])
    first = [plan.perm.clone(), plan.chunk_start[:n].clone(), plan.chunk_len[:n].clone(),
             plan.chunk_adapter[:n].clone(), plan.counters.clone(), plan.work.clone()]
    plan_decode(tok, pool, group=4, out=plan)
    torch.cuda.synchronize()
    second = [plan.perm, plan.chunk_start[:n], plan.chunk_len[:n], plan.chunk_adapter[:n], plan.counters, plan.work]
    for a, b in zip(first, second):
        assert torch.equal(a, b)
