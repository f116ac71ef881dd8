"""GPU parity of the adapter swap-in: the scatter kernel through the C ABI is a bit-exact copy onto
the slot's pages (checked against the oracle), and an adapter loaded through AdapterLoader gives the
same LoRA result as the oracle on the same weights."""
import ctypes as C

import numpy as np
import pytest
import torch

from gpu_common import assert_close_bits, say
from helpers import FP16, bits_of, torch_to_bits
from mlora import AdapterLoader, AdapterPool, _ext, bgmv, layer_order, plan_decode
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rank,page_rows,widths", [(16, 8, [4096, 4096]), (5, 8, [64, 24, 4096]), (64, 8, [11008, 4096, 40]),
                                                   (33, 16, [72]), (1, 1, [8, 16])])
def test_scatter_is_a_bit_exact_copy(rank, page_rows, widths):
    rng = np.random.default_rng(rank * 100 + page_rows)
    n_pages = 29
    need = -(-rank // page_rows)
    pages = rng.permutation(n_pages)[:need].astype(np.int32)
    srcs = [rng.integers(0, 65536, (rank, w)).astype(np.uint16) for w in widths]
    slabs = [rng.integers(0, 65536, (n_pages * page_rows, w)).astype(np.uint16) for w in widths]
    want = [orc.pool_scatter(s, d.copy(), pages, page_rows) for s, d in zip(srcs, slabs)]
    d_src = [torch.from_numpy(s.view(np.int16)).cuda() for s in srcs]
    d_dst = [torch.from_numpy(d.view(np.int16)).cuda() for d in slabs]
    n = len(widths)
    src, dst, wid = (C.c_void_p * 16)(), (C.c_void_p * 16)(), (C.c_int32 * 16)()
    for i in range(n):
        src[i], dst[i], wid[i] = d_src[i].data_ptr(), d_dst[i].data_ptr(), widths[i]
    say(f"scatter rank={rank} page_rows={page_rows} widths={widths}")
    rc = _ext.lib().mlora_pool_scatter(n, src, dst, wid, (C.c_int32 * need)(*pages.tolist()), need, rank, page_rows,
                                       n_pages, 2, torch.cuda.current_stream().cuda_stream)
    _ext.check(rc)
    torch.cuda.synchronize()
    for i in range(n):
        assert np.array_equal(d_dst[i].cpu().numpy().view(np.uint16), want[i])


def test_loader_end_to_end():
    rng = np.random.default_rng(5)
    L, H, HO = 6, 512, 768
    projections = {"q": (H, HO), "k": (H, H), "v": (H, H)}
    pool = AdapterPool(L, projections, n_slots=6, n_pages=24, page_rows=8, max_rank=32, dtype=torch.float16, device="cuda")
    # poison the slabs: anything the loader does not write must stay as it is
    for t in list(pool.a_rows.values()) + list(pool.b_rows.values()):
        t.fill_(7.0)
    loader = AdapterLoader(pool, layers_per_copy=2, first_layer=2)
    assert loader.stream.priority == 0
    adapters = {}
    for slot, rank in ((4, 16), (1, 24), (2, 5)):
        w = {p: (torch.from_numpy((rng.standard_normal((L, hin, rank)) * 0.05).astype(np.float32)),
                 torch.from_numpy((rng.standard_normal((L, rank, hout)) * 0.05).astype(np.float32)))
             for p, (hin, hout) in projections.items()}
        host = loader.stage(w, rank, 32.0 / rank)
        assert host.blob.is_pinned() and host.blob.shape == (L, rank * (3 * H + HO + 2 * H))
        say(f"loader: slot {slot} rank {rank}")
        ticket = loader.load_async(slot, host)
        assert ticket.order == layer_order(L, 2) == [2, 3, 4, 5, 0, 1]
        ticket.wait()
        assert all(ticket.ready(layer) for layer in range(L)) and ticket.progress() == 0 and ticket.layers_ready() == L
        assert ticket.use_gpu_pipeline(0)
        adapters[slot] = (rank, w)
    torch.cuda.synchronize()
    # every slab row: the loaded value where an adapter owns it, the poison elsewhere
    for p, (hin, hout) in projections.items():
        for layer in range(L):
            want_a = np.full((24 * 8, hin), 7.0, np.float16)
            want_b = np.full((24 * 8, hout), 7.0, np.float16)
            for slot, (rank, w) in adapters.items():
                rows = pool.rows_of(slot).cpu().numpy()
                want_a[rows] = w[p][0][layer].numpy().T.astype(np.float16)
                want_b[rows] = w[p][1][layer].numpy().astype(np.float16)
            assert np.array_equal(pool.a_rows[p][layer].cpu().numpy().view(np.uint16), want_a.view(np.uint16))
            assert np.array_equal(pool.b_rows[p][layer].cpu().numpy().view(np.uint16), want_b.view(np.uint16))
    # and the decode kernel reads them in place: compare with the oracle on the same weights
    T, layer = 33, 3
    tok = rng.choice([4, 1, 2, -1], size=T).astype(np.int32)
    x = bits_of(rng.standard_normal((T, H)).astype(np.float32), FP16)
    y0 = bits_of(rng.standard_normal((T, HO)).astype(np.float32), FP16)
    t = torch.from_numpy(tok).cuda()
    xt = torch.from_numpy(x.view(np.int16)).cuda().view(torch.float16)
    yt = torch.from_numpy(y0.view(np.int16)).cuda().view(torch.float16)
    # a consumer stream that waits on the device for the layer it reads (no host synchronisation)
    host = loader.stage(adapters[4][1], 16, 2.0)
    ticket = loader.load_async(4, host)                              # reload slot 4 (same weights, new pages)
    ticket.wait_layer(layer)
    bgmv([yt], [xt], pool, layer, ["q"], t, plan=plan_decode(t, pool, group=4))
    torch.cuda.synchronize()
    a_np = pool.a_rows["q"][layer].cpu().numpy().view(np.uint16)
    b_np = pool.b_rows["q"][layer].cpu().numpy().view(np.uint16)
    want = orc.lora_apply_paged(x, a_np, b_np, tok, pool.h_page_tbl, pool.h_page_tbl, pool.h_rank, pool.h_scaling,
                                pool.page_rows, FP16, y0=y0)
    assert_close_bits(torch_to_bits(yt), want, FP16, "bgmv on loaded adapters")


def test_scatter_rejects_bad_arguments():
    lib = _ext.lib()
    buf = torch.zeros(1024, dtype=torch.int16, device="cuda")
    src, dst, wid = (C.c_void_p * 16)(), (C.c_void_p * 16)(), (C.c_int32 * 16)()
    src[0], dst[0], wid[0] = buf.data_ptr(), buf.data_ptr(), 8
    pages = (C.c_int32 * 2)(0, 99)
    assert lib.mlora_pool_scatter(1, src, dst, wid, pages, 2, 16, 8, 4, 2, None) == _ext.MLORA_ERANGE      # page 99 of 4
    assert lib.mlora_pool_scatter(1, src, dst, wid, pages, 1, 16, 8, 4, 2, None) == _ext.MLORA_ERANGE      # too few pages
    wid[0] = 4
    assert lib.mlora_pool_scatter(1, src, dst, wid, pages, 1, 8, 8, 4, 2, None) == _ext.MLORA_EALIGN       # 8-byte rows
    assert lib.mlora_pool_scatter(17, src, dst, wid, pages, 1, 8, 8, 4, 2, None) == _ext.MLORA_ERANGE
