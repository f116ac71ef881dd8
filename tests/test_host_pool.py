"""Host logic of the paged adapter pool (page table bookkeeping), on CPU tensors."""
import numpy as np
import pytest
import torch

from mlora.pool import AdapterPool


def _pool(**kw):
    a = dict(n_layers=2, projections={"q": (64, 64), "down": (128, 64)}, n_slots=6, n_pages=10, page_rows=8,
             max_rank=64, dtype=torch.float16, device="cpu")
    a.update(kw)
    return AdapterPool(**a)


def test_allocate_release_accounting():
    p = _pool()
    assert p.free_pages == 10 and p.max_pages == 8
    pg = p.allocate(0, 16, 2.0)
    assert len(pg) == 2 and p.free_pages == 8
    p.allocate(1, 64, 0.5)
    assert p.free_pages == 0
    with pytest.raises(MemoryError):
        p.allocate(2, 8, 1.0)
    p.release(0)
    assert p.free_pages == 2 and p.h_rank[0] == 0 and np.all(p.h_page_tbl[0] == -1)
    p.allocate(2, 9, 1.0)                      # rank 9 needs two pages
    assert p.free_pages == 0
    used = np.concatenate([p.h_page_tbl[1, :8], p.h_page_tbl[2, :2]])
    assert len(set(used.tolist())) == 10       # no page handed out twice
    p.sync()
    assert torch.equal(p.page_tbl, torch.from_numpy(p.h_page_tbl))
    assert torch.equal(p.rank, torch.from_numpy(p.h_rank))


def test_explicit_pages_and_errors():
    p = _pool()
    p.allocate(3, 24, 1.0, pages=[9, 0, 4])
    assert p.h_page_tbl[3, :3].tolist() == [9, 0, 4]
    with pytest.raises(ValueError):
        p.allocate(4, 8, 1.0, pages=[9])       # in use
    with pytest.raises(ValueError):
        p.allocate(4, 16, 1.0, pages=[1])      # wrong count
    with pytest.raises(ValueError):
        p.allocate(4, 65, 1.0)
    with pytest.raises(IndexError):
        p.allocate(6, 8, 1.0)
    with pytest.raises(ValueError):
        _pool(page_rows=3)


def test_move_is_a_table_update():
    p = _pool()
    p.allocate(0, 32, 1.0)
    before = p.h_page_tbl[0].copy()
    free = p.free_pages
    p.move(0, 5)
    assert np.array_equal(p.h_page_tbl[5], before) and p.h_rank[5] == 32 and p.h_rank[0] == 0
    assert p.free_pages == free


def test_move_rejects_bad_arguments_and_evicts_the_destination():
    p = _pool()
    p.allocate(0, 32, 1.0)
    p.allocate(1, 8, 2.0)
    snap = (p.h_page_tbl.copy(), p.h_rank.copy(), p.free_pages)
    with pytest.raises(ValueError):
        p.move(0, 0)                           # would free the adapter's own pages
    with pytest.raises(ValueError):
        p.move(3, 1)                           # empty source would silently evict slot 1
    with pytest.raises(IndexError):
        p.move(0, 6)
    with pytest.raises(IndexError):
        p.move(-1, 2)
    with pytest.raises(IndexError):
        p.release(6)
    assert np.array_equal(p.h_page_tbl, snap[0]) and np.array_equal(p.h_rank, snap[1]) and p.free_pages == snap[2]
    pages0 = p.h_page_tbl[0].copy()
    p.move(0, 1)                               # occupied destination: its adapter is evicted, its page returns
    assert p.free_pages == snap[2] + 1 and p.h_rank[1] == 32 and p.h_rank[0] == 0
    assert np.array_equal(p.h_page_tbl[1], pages0)


def test_load_places_rank_rows_on_the_adapters_pages():
    p = _pool()
    p.allocate(1, 16, 2.0, pages=[7, 2])
    A = torch.randn(128, 16)
    B = torch.randn(16, 64)
    p.load(1, 1, "down", A, B)
    rows = p.rows_of(1)
    assert rows.tolist() == list(range(56, 64)) + list(range(16, 24))
    assert torch.equal(p.a_rows["down"][1][rows], A.t().to(torch.float16))
    assert torch.equal(p.b_rows["down"][1][rows], B.to(torch.float16))
    assert p.a_rows["down"][0].abs().sum() == 0          # other layer untouched
    with pytest.raises(ValueError):
        p.load(1, 1, "q", A, B)
