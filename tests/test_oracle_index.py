"""Pins the oracle's integer work (gather, grouping, work lists, chunk plan) against numpy closed
forms and brute force.  None of these re-type the oracle's loops: they use argsort / unique /
explicit enumeration."""
import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from oracle import oracle as orc


def _np_gather(tok, page_tbl, rank, scaling, page_rows):
    T = len(tok)
    N, mp = page_tbl.shape
    valid = tok >= 0
    a = np.where(valid, tok, 0)
    r = np.where(valid, rank[a], 0)
    npg = -(-r // page_rows)
    p = np.arange(mp)[None, :]
    off = np.where(valid[:, None] & (p < npg[:, None]), page_tbl[a] * page_rows, -1)
    return off.astype(np.int32), r.astype(np.int32), np.where(valid, scaling[a], 0).astype(np.float32)


@pytest.mark.parametrize("page_rows", [1, 8, 16])
def test_pool_gather_closed_form(page_rows):
    rng = np.random.default_rng(page_rows)
    N, T = 37, 300
    rank = rng.choice([1, 3, 8, 16, 24, 32, 64], N).astype(np.int32)
    mp = -(-64 // page_rows)
    page_tbl = rng.integers(0, 5000, (N, mp)).astype(np.int32)
    scaling = rng.random(N).astype(np.float32)
    tok = rng.integers(-1, N, T).astype(np.int32)
    got = orc.pool_gather(tok, page_tbl, rank, scaling, page_rows)
    want = _np_gather(tok, page_tbl, rank, scaling, page_rows)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


def test_pool_gather_rejects_out_of_range():
    page_tbl = np.zeros((4, 2), np.int32)
    with pytest.raises(IndexError):
        orc.pool_gather(np.array([0, 4], np.int32), page_tbl, np.ones(4, np.int32), np.ones(4, np.float32), 8)
    with pytest.raises(IndexError):   # rank needs more pages than the table has
        orc.pool_gather(np.array([0], np.int32), page_tbl, np.full(4, 17, np.int32), np.ones(4, np.float32), 8)


def _np_segments(tok, n_adapters):
    key = np.where(tok >= 0, tok, n_adapters)
    perm = np.argsort(key, kind="stable").astype(np.int32)
    valid = tok[tok >= 0]
    ad, cnt = np.unique(valid, return_counts=True)
    start = np.concatenate([[0], np.cumsum(cnt)[:-1]]) if len(cnt) else np.zeros(0)
    return perm, start.astype(np.int32), cnt.astype(np.int32), ad.astype(np.int32), len(valid)


@settings(max_examples=200, deadline=None)
@given(st.lists(st.integers(-1, 11), min_size=0, max_size=80))
def test_build_segments_vs_argsort(toks):
    tok = np.array(toks, np.int32)
    perm, ss, sl, sa, nv = orc.build_segments(tok, 12)
    wperm, wss, wsl, wsa, wnv = _np_segments(tok, 12)
    assert np.array_equal(perm, wperm) and np.array_equal(ss, wss) and np.array_equal(sl, wsl)
    assert np.array_equal(sa, wsa) and nv == wnv


def test_build_segments_empty_and_single():
    perm, ss, sl, sa, nv = orc.build_segments(np.zeros(0, np.int32), 4)
    assert perm.size == 0 and ss.size == 0 and nv == 0
    perm, ss, sl, sa, nv = orc.build_segments(np.array([3], np.int32), 4)
    assert perm.tolist() == [0] and ss.tolist() == [0] and sl.tolist() == [1] and sa.tolist() == [3] and nv == 1
    with pytest.raises(IndexError):
        orc.build_segments(np.array([4], np.int32), 4)


@settings(max_examples=150, deadline=None)
@given(st.lists(st.integers(-1, 6), min_size=0, max_size=60), st.sampled_from([1, 2, 4, 8]))
def test_build_chunks_brute_force(toks, group):
    tok = np.array(toks, np.int32)
    T = len(tok)
    perm, ss, sl, sa, nv = orc.build_segments(tok, 7)
    cs, cl, ca = orc.build_chunks(ss, sl, sa, nv, T, group)
    # brute force over sorted positions: a new chunk starts when the adapter changes or the
    # running chunk already holds `group` tokens
    key = [int(tok[p]) if tok[p] >= 0 else -1 for p in perm]
    want = []
    for i, k in enumerate(key):
        if want and want[-1][2] == k and want[-1][1] < group:
            want[-1][1] += 1
        else:
            want.append([i, 1, k])
    assert [list(map(int, c)) for c in zip(cs, cl, ca)] == want
    assert int(cl.sum()) == T
    assert len(cs) <= max(T, 1)


def _record_order(ca, rank, P, heavy_first):
    """Chunk held by every position of the record sequence: chunk order, and for batches of at most 2048 tokens
    falling rank inside each range of P chunks (one XCD), ties in chunk order (numpy's stable argsort)."""
    n = len(ca)
    crk = np.array([min(max(int(rank[a]), 0), 64) if a >= 0 else 0 for a in ca], dtype=np.int64)
    order = []
    for lo in range(0, n, max(P, 1)):
        idx = np.arange(lo, min(lo + P, n))
        order += list(idx[np.argsort(-crk[idx], kind="stable")] if heavy_first else idx)
    return order


def test_build_work_by_enumeration():
    """Work records: position pos of the record sequence sits at b = (pos mod P) * 8 + pos // P; which chunk a
    position holds (see _record_order) and the contents, checked field by field."""
    rng = np.random.default_rng(8)
    N, T, group, page_rows, n_pages = 9, 45, 4, 8, 40
    rank = rng.choice([8, 16, 24, 64], N).astype(np.int32)
    page_tbl = rng.integers(0, n_pages, (N, 8)).astype(np.int32)
    page_tbl[3, 1] = n_pages + 5                  # a page id outside the slab -> rows marked absent
    scaling = rng.random(N).astype(np.float32)
    tok = rng.integers(-1, N, T).astype(np.int32)
    perm, ss, sl, sa, nv = orc.build_segments(tok, N)
    cs, cl, ca = orc.build_chunks(ss, sl, sa, nv, T, group)
    work = orc.build_work(cs, cl, ca, perm, page_tbl, rank, scaling, page_rows, n_pages, T)
    cap = ((T + 7) // 8) * 8
    assert work.shape == (cap, orc.WORK_WORDS)
    P = -(-len(cs) // 8)
    used = set()
    order = _record_order(ca, rank, P, heavy_first=True)
    assert sorted(order) == list(range(len(cs)))
    # heavy first inside a range, and a range keeps its chunks (one XCD, residue pos // P)
    for pos in range(1, len(order)):
        if pos % P:
            ra, rb = (rank[ca[order[k]]] if ca[order[k]] >= 0 else 0 for k in (pos - 1, pos))
            assert ra >= rb
    assert all(order[pos] // P == pos // P for pos in range(len(order)))
    for pos, c in enumerate(order):
        b = (pos % P) * 8 + pos // P
        used.add(b)
        w = work[b]
        a = int(ca[c])
        assert w[0] == cl[c] and w[1] == a
        assert w[4:4 + cl[c]].tolist() == perm[cs[c]:cs[c] + cl[c]].tolist() and np.all(w[4 + cl[c]:12] == -1)
        assert np.all(w[12:16] == 0)
        if a < 0:
            assert w[2] == 0 and w[3] == 0 and np.all(w[16:] == -1)
            continue
        assert w[2] == rank[a] and w[3] == scaling[a:a + 1].view(np.int32)[0]
        for j in range(64):
            pg = page_tbl[a, j // page_rows]
            want = pg * page_rows + j % page_rows if (j < rank[a] and 0 <= pg < n_pages) else -1
            assert w[16 + j] == want
    # consecutive positions of a range share blockIdx mod 8 (one XCD): position pos sits at residue pos // P
    assert all(((pos % P) * 8 + pos // P) % 8 == pos // P for pos in range(len(cs)))
    for b in range(cap):
        if b not in used:
            assert work[b, 0] == 0 and work[b, 1] == -1 and np.all(work[b, 2:] == 0)


def test_build_work_keeps_chunk_order_beyond_2048_tokens():
    rng = np.random.default_rng(9)
    N, T, group, page_rows, n_pages = 40, 2100, 4, 8, 400
    rank = rng.choice([8, 16, 32, 64], N).astype(np.int32)
    page_tbl = rng.integers(0, n_pages, (N, 8)).astype(np.int32)
    scaling = rng.random(N).astype(np.float32)
    tok = rng.integers(0, N, T).astype(np.int32)
    perm, ss, sl, sa, nv = orc.build_segments(tok, N)
    cs, cl, ca = orc.build_chunks(ss, sl, sa, nv, T, group)
    work = orc.build_work(cs, cl, ca, perm, page_tbl, rank, scaling, page_rows, n_pages, T)
    P = -(-len(cs) // 8)
    for c in range(len(cs)):
        w = work[(c % P) * 8 + c // P]
        assert w[0] == cl[c] and w[1] == ca[c] and w[4] == perm[cs[c]]


def test_sgmv_plan_brute_force():
    rng = np.random.default_rng(5)
    lens = rng.integers(0, 400, 23)
    starts = np.concatenate([[0], np.cumsum(lens)[:-1]])
    ts, t0, tn = orc.sgmv_plan(starts, lens, 64)
    want = [(s, int(starts[s]) + o, min(64, int(lens[s]) - o)) for s in range(23) for o in range(0, int(lens[s]), 64)]
    assert list(zip(ts.tolist(), t0.tolist(), tn.tolist())) == want
    covered = np.zeros(int(lens.sum()), int)
    for _, a, n in want:
        covered[a:a + n] += 1
    assert np.all(covered == 1)


def test_sgmv_plan_aligned_brute_force():
    """Aligned cuts: every token of every segment in exactly one tile, no tile crosses a multiple of 64 or a
    segment end, tiles in token order within a segment, and as few tiles as that allows."""
    rng = np.random.default_rng(6)
    lens = rng.integers(0, 400, 29)
    gaps = rng.integers(0, 3, 29) * rng.integers(0, 70, 29)
    starts = np.cumsum(gaps) + np.concatenate([[0], np.cumsum(lens)[:-1]])
    ts, t0, tn = orc.sgmv_plan(starts, lens, 64, aligned=True)
    want = []
    for s in range(29):
        toks = np.arange(int(starts[s]), int(starts[s] + lens[s]))
        for k in np.unique(toks // 64):                       # ascending
            part = toks[toks // 64 == k]
            want.append((s, int(part[0]), len(part)))
    assert list(zip(ts.tolist(), t0.tolist(), tn.tolist())) == want
    assert all(a // 64 == (a + n - 1) // 64 and 1 <= n <= 64 for _, a, n in want)
    # never more than one tile more per segment end than the unaligned cut
    assert len(want) <= len(orc.sgmv_plan(starts, lens, 64)[0]) + int((lens > 0).sum())


@pytest.mark.parametrize("batch,tkn,cap", [(1, 64, 8), (3, 20, 8), (2, 8, 8), (4, 1, 16), (2, 17, 16), (1, 256, 8)])
def test_cpu_chunk_plan_matches_reference_formulas(batch, tkn, cap):
    req, tok0, ntok = orc.cpu_chunk_plan(batch, tkn, cap)
    # lightllm/models/lora_cpu.py:150-151,210-213: cpu_per_request and the last chunk's size
    cpr = (tkn - 1) // cap + 1
    last = tkn % cap if tkn % cap > 0 else cap
    assert len(req) == batch * cpr
    for row_id in range(batch * cpr):
        b, off = divmod(row_id, cpr)             # app.py:133-134 dim_0, dim_1
        assert req[row_id] == b and tok0[row_id] == off * cap
        assert ntok[row_id] == (last if off == cpr - 1 else cap)
    cover = np.zeros((batch, tkn), int)
    for b, a, n in zip(req, tok0, ntok):
        cover[b, a:a + n] += 1
    assert np.all(cover == 1)


def test_pool_scatter_is_a_fancy_index_assignment():
    rng = np.random.default_rng(77)
    for rank, page_rows, width in [(16, 8, 64), (5, 8, 24), (64, 8, 40), (9, 4, 16), (1, 1, 8), (33, 16, 72)]:
        n_pages = 23
        need = -(-rank // page_rows)
        pages = rng.permutation(n_pages)[:need + 1].astype(np.int32)       # one spare entry that must not be used
        src = rng.integers(0, 65536, (rank, width)).astype(np.uint16)
        slab = rng.integers(0, 65536, (n_pages * page_rows, width)).astype(np.uint16)
        want = slab.copy()
        k = np.arange(rank)
        want[pages[k // page_rows] * page_rows + k % page_rows] = src
        got = orc.pool_scatter(src, slab.copy(), pages, page_rows)
        assert np.array_equal(got, want)
    with pytest.raises(IndexError):
        orc.pool_scatter(src, slab.copy(), np.array([0, 99], np.int32), 16)          # page id outside the slab
    with pytest.raises(IndexError):
        orc.pool_scatter(src, slab.copy(), np.array([0], np.int32), 16)              # too few pages for the rank
