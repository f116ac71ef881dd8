"""Known-answer files under tests/golden/: the CPU checker must still reproduce them bit for bit
(CPU), and the HIP kernels must meet them through the C ABI (GPU)."""
import os

import numpy as np
import pytest

from oracle import oracle as orc

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    return dict(np.load(os.path.join(G, name), allow_pickle=False))


@pytest.mark.parametrize("name", ["apply_fp16.npz", "apply_bf16.npz"])
def test_oracle_reproduces_apply(name):
    d = _load(name)
    args = (d["x"], d["a_rows"], d["b_rows"], d["tok"], d["page_tbl"], d["page_tbl"], d["rank"], d["scaling"],
            int(d["page_rows"]), int(d["dtype"]))
    assert np.array_equal(orc.lora_apply_paged(*args, y0=d["y0"]), d["y_acc"])
    assert np.array_equal(orc.lora_apply_paged(*args, y0=None), d["y_delta"])


def test_oracle_reproduces_gather():
    d = _load("gather.npz")
    N = len(d["rank"])
    perm, ss, sl, sa, nv = orc.build_segments(d["tok"], N)
    cs, cl, ca = orc.build_chunks(ss, sl, sa, nv, len(d["tok"]), int(d["group"]))
    ro, rk, sc = orc.pool_gather(d["tok"], d["page_tbl"], d["rank"], d["scaling"], int(d["page_rows"]))
    work = orc.build_work(cs, cl, ca, perm, d["page_tbl"], d["rank"], d["scaling"], int(d["page_rows"]), int(d["n_pages"]),
                          len(d["tok"]))
    assert np.array_equal(work, d["work"])
    for got, key in ((perm, "perm"), (ss, "seg_start"), (sl, "seg_len"), (sa, "seg_adapter"), (cs, "chunk_start"),
                     (cl, "chunk_len"), (ca, "chunk_adapter"), (ro, "row_off"), (rk, "tok_rank")):
        assert np.array_equal(got, d[key]), key
    assert nv == int(d["n_valid"]) and np.array_equal(sc.view(np.uint32), d["tok_scale"].view(np.uint32))


def test_oracle_reproduces_reflayout():
    d = _load("reflayout.npz")
    y = d["y0"].copy()
    orc.add_lora_bgmv_ref(y, d["x"], d["wa"], d["wb"], d["idx"], int(d["layer"]), 1.0)
    assert np.array_equal(y, d["y"])
    assert np.array_equal(orc.prefill_bmm_ref(d["xp"], d["wa"][:3], d["wb"][:3], int(d["layer"]), orc.FP16), d["yp"])


# ------------------------------------------------------------------ GPU
@pytest.mark.gpu
@pytest.mark.parametrize("name", ["apply_fp16.npz", "apply_bf16.npz"])
@pytest.mark.parametrize("group", [0, 4])
def test_gpu_apply_meets_golden(name, group):
    import torch
    from gpu_common import assert_close_bits, say, tdtype
    from helpers import bits_to_torch, torch_to_bits
    from mlora import AdapterPool, bgmv, plan_decode, sgmv
    d = _load(name)
    dtype, page_rows = int(d["dtype"]), int(d["page_rows"])
    N = len(d["rank"])
    hin, hout = d["a_rows"].shape[1], d["b_rows"].shape[1]
    pool = AdapterPool(1, {"p": (hin, hout)}, N, d["a_rows"].shape[0] // page_rows, page_rows=page_rows, max_rank=64,
                       dtype=tdtype(dtype), device="cuda")
    pool.h_page_tbl[:, :d["page_tbl"].shape[1]] = d["page_tbl"]
    pool.h_rank[:] = d["rank"]
    pool.h_scaling[:] = d["scaling"]
    pool._dirty = True
    pool.sync()
    pool.a_rows["p"][0].copy_(bits_to_torch(d["a_rows"], dtype))
    pool.b_rows["p"][0].copy_(bits_to_torch(d["b_rows"], dtype))
    tok = torch.from_numpy(d["tok"]).cuda()
    x = bits_to_torch(d["x"], dtype, "cuda")
    y = bits_to_torch(d["y0"], dtype, "cuda")
    say(f"golden {name} bgmv group={group}")
    bgmv([y], [x], pool, 0, ["p"], tok, plan=plan_decode(tok, pool, group=group) if group else None)
    yd = torch.zeros_like(y)
    bgmv([yd], [x], pool, 0, ["p"], tok, accumulate=False)
    torch.cuda.synchronize()
    assert_close_bits(torch_to_bits(y), d["y_acc"], dtype)
    assert_close_bits(torch_to_bits(yd), d["y_delta"], dtype)
    if group:
        # the same tokens as one-token segments through the prefill kernels
        T = len(d["tok"])
        ys = bits_to_torch(d["y0"], dtype, "cuda")
        say(f"golden {name} sgmv, one segment per token")
        sgmv(ys, x, pool, 0, "p", torch.arange(T, dtype=torch.int32, device="cuda"),
             torch.ones(T, dtype=torch.int32, device="cuda"), tok)
        torch.cuda.synchronize()
        assert_close_bits(torch_to_bits(ys), d["y_acc"], dtype)


@pytest.mark.gpu
def test_gpu_gather_meets_golden():
    import torch
    from gpu_common import say
    from mlora import AdapterPool, _ext, plan_decode
    d = _load("gather.npz")
    N, page_rows, group = len(d["rank"]), int(d["page_rows"]), int(d["group"])
    pool = AdapterPool(1, {"p": (64, 64)}, N, int(d["n_pages"]), page_rows=page_rows, max_rank=64, device="cuda")
    pool.h_page_tbl[:] = d["page_tbl"]
    pool.h_rank[:] = d["rank"]
    pool.h_scaling[:] = d["scaling"]
    pool._dirty = True
    say("golden gather")
    plan = plan_decode(torch.from_numpy(d["tok"]).cuda(), pool, group=group, per_token=True)
    torch.cuda.synchronize()
    cnt = plan.counters.cpu().numpy()
    ns, nc = len(d["seg_start"]), len(d["chunk_start"])
    assert cnt[_ext.CNT_NSEG] == ns and cnt[_ext.CNT_NCHUNK] == nc and cnt[_ext.CNT_NVALID] == int(d["n_valid"])
    for got, key, n in ((plan.perm, "perm", None), (plan.seg_start, "seg_start", ns), (plan.seg_len, "seg_len", ns),
                        (plan.seg_adapter, "seg_adapter", ns), (plan.chunk_start, "chunk_start", nc),
                        (plan.chunk_len, "chunk_len", nc), (plan.chunk_adapter, "chunk_adapter", nc),
                        (plan.row_off, "row_off", None), (plan.tok_rank, "tok_rank", None)):
        assert np.array_equal(got.cpu().numpy()[:n], d[key]), key
    assert np.array_equal(plan.tok_scale.cpu().numpy().view(np.uint32), d["tok_scale"].view(np.uint32))
    assert np.array_equal(plan.work.cpu().numpy(), d["work"])


@pytest.mark.gpu
def test_gpu_reflayout_meets_golden():
    import torch
    from gpu_common import assert_close_bits, say
    from helpers import FP16, bits_to_torch, torch_to_bits
    from mlora import add_lora_bgmv, lora_prefill_ref
    d = _load("reflayout.npz")
    wa, wb = bits_to_torch(d["wa"], FP16, "cuda"), bits_to_torch(d["wb"], FP16, "cuda")
    y = bits_to_torch(d["y0"], FP16, "cuda")
    say("golden reflayout decode + prefill")
    add_lora_bgmv(y, bits_to_torch(d["x"], FP16, "cuda"), wa, wb, torch.from_numpy(d["idx"]).cuda(), int(d["layer"]), 1.0)
    yp = lora_prefill_ref(bits_to_torch(d["xp"], FP16, "cuda"), wa, wb, int(d["layer"]))
    torch.cuda.synchronize()
    assert_close_bits(torch_to_bits(y), d["y"], FP16)
    assert_close_bits(torch_to_bits(yp), d["yp"], FP16)
