"""HIP graph replays of the decode and prefill steps give the eager results bit for bit, replay after
replay, with eager work and synchronisations in between (nothing in the library records a memset node
or allocates during capture once the plan's buffers exist)."""
import numpy as np
import pytest
import torch

from gpu_common import say, upload_pool
from helpers import FP16, PagedPool
from mlora import bgmv, plan_decode, plan_prefill, sgmv_multi

pytestmark = pytest.mark.gpu


def test_graph_replays_match_eager():
    rng = np.random.default_rng(91)
    ranks = [16, 8, 32, 64, 24, 16]
    H = 512
    pp = PagedPool(rng, ranks, H, H, page_rows=8, dtype=FP16)
    pool = upload_pool(pp, projections={"p": (H, H), "o": (H, H)})
    pool.a_rows["o"][0].normal_(0, 0.02)
    pool.b_rows["o"][0].normal_(0, 0.02)
    T = 97
    tok = torch.from_numpy(rng.integers(-1, len(ranks), T).astype(np.int32)).cuda()
    lens = np.array([40, 7, 50], np.int32)
    ss = torch.from_numpy(np.array([0, 40, 47], np.int32)).cuda()
    sl = torch.from_numpy(lens).cuda()
    sa = torch.from_numpy(np.array([3, 0, 5], np.int32)).cuda()
    x = torch.randn(T, H, device="cuda").half()
    y_dec = [torch.zeros(T, H, device="cuda").half() for _ in range(2)]
    y_pre = [torch.zeros(T, H, device="cuda").half() for _ in range(2)]
    y0 = torch.randn(T, H, device="cuda").half()
    plan = plan_decode(tok, pool, group=4)
    pplan = plan_prefill(ss, sl, sa, T, pool, n_proj=2)

    def step():
        for y in y_dec + y_pre:
            y.copy_(y0)
        plan_decode(tok, pool, out=plan)
        bgmv(y_dec, [x, x], pool, 0, ["p", "o"], tok, plan=plan)
        plan_prefill(ss, sl, sa, T, pool, workspace=pplan.workspace, n_proj=2)
        sgmv_multi(y_pre, [x, x], pool, 0, ["p", "o"], pplan)

    say("graph: eager reference step")
    step()                                        # also allocates the plan's intermediate buffer
    torch.cuda.synchronize()
    want = [t.clone() for t in y_dec + y_pre]
    assert not torch.equal(want[0], y0)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    for rep in range(4):
        # eager work of the program itself between the replays
        for t in y_dec + y_pre:
            t.fill_(float(rep))
        scratch = (torch.randn(1 << 20, device="cuda") * 2).sum()
        torch.cuda.synchronize()
        say(f"graph: replay {rep}")
        g.replay()
        torch.cuda.synchronize()
        assert scratch.isfinite()
        for got, w in zip(y_dec + y_pre, want):
            assert torch.equal(got, w), rep


def test_graph_replays_of_the_one_pass_projection_match_eager():
    """The base projection + LoRA call (plan, shrink, scaled reduce, GEMM) under a HIP graph: every replay gives the
    eager result bit for bit, with eager work in between."""
    from mlora import gemm_lora
    rng = np.random.default_rng(92)
    ranks = [16, 64, 32]
    hin, hout = 320, 520
    pp = PagedPool(rng, ranks, hin, hout, page_rows=8, dtype=FP16)
    pool = upload_pool(pp)
    lens = np.array([130, 7, 200, 64], np.int32)
    starts = np.array([2, 132, 140, 345], np.int32)
    T = 420
    ss, sl = torch.from_numpy(starts).cuda(), torch.from_numpy(lens).cuda()
    sa = torch.from_numpy(np.array([1, -1, 0, 2], np.int32)).cuda()
    x = torch.randn(T, hin, device="cuda").half()
    w = (torch.randn(hin, hout, device="cuda") / hin ** 0.5).half()
    y = torch.zeros(T, hout, device="cuda").half()
    pplan = plan_prefill(ss, sl, sa, T, pool, aligned=True)

    def step():
        plan_prefill(ss, sl, sa, T, pool, workspace=pplan.workspace, aligned=True)
        gemm_lora([y], [x], [w], pool, 0, ["p"], pplan)

    say("graph: eager one-pass projection")
    step()
    torch.cuda.synchronize()
    want = y.clone()
    assert bool(torch.isfinite(want.float()).all()) and not torch.equal(want, torch.mm(x, w))   # the delta is in there
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    for rep in range(4):
        y.fill_(float(rep))
        scratch = (torch.randn(1 << 20, device="cuda") * 2).sum()
        torch.cuda.synchronize()
        say(f"graph: one-pass projection replay {rep}")
        g.replay()
        torch.cuda.synchronize()
        assert scratch.isfinite()
        assert torch.equal(y, want), rep


@pytest.mark.parametrize("size", ["one round (config 2 shape)", "many rounds (config 5 layer)"])
def test_graph_replay_follows_a_changed_batch(size):
    """A captured decode step (gather + BGMV) reads its token -> adapter vector from device memory: when the caller
    overwrites that vector between replays, the replay must use the new grouping -- the work records are rewritten by
    the gather node and read by the decode kernels of the same replay (header words through scalar loads), so a stale
    copy anywhere would show here.  Each replay is compared bit for bit with an eager run on the same batch."""
    from mlora import workloads
    if size.startswith("one"):
        shapes, T, N, rank, alpha = workloads.LLAMA7B_ATTN, 256, 64, 16, 1.0
    else:
        shapes, T, N, rank, alpha = workloads.LLAMA7B_ALL, 512, 1000, 32, 1.1
    names = list(shapes)
    wl = workloads.make_decode("graph", shapes, 1, T, N, [rank], alpha, seed=77, device="cuda")
    pool = wl.pool
    rng = np.random.default_rng(5)
    batches = [wl.tok_adapter,
               workloads.zipf_adapters(rng, T, N, 0.6),
               np.where(rng.random(T) < 0.1, -1, workloads.zipf_adapters(rng, T, N, 1.4)).astype(np.int32)]
    tok = torch.from_numpy(batches[0].copy()).cuda()
    gen = torch.Generator(device="cuda").manual_seed(3)
    xs = {h: torch.randn(T, h, device="cuda", generator=gen).half() for h in {s[0] for s in shapes.values()}}
    y0 = [torch.randn(T, shapes[p][1], device="cuda", generator=gen).half() for p in names]
    ys = [t.clone() for t in y0]
    plan = plan_decode(tok, pool, group=4)

    def step():
        for y, src in zip(ys, y0):
            y.copy_(src)
        plan_decode(tok, pool, out=plan)
        bgmv(ys, [xs[shapes[p][0]] for p in names], pool, 0, names, tok, plan=plan, fused=False)

    want = []
    for bt in batches:
        tok.copy_(torch.from_numpy(bt))
        step()
        torch.cuda.synchronize()
        want.append([t.clone() for t in ys])
    assert not torch.equal(want[0][0], want[1][0])
    tok.copy_(torch.from_numpy(batches[0]))
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    for rep, which in enumerate([0, 1, 2, 1, 0, 2]):
        tok.copy_(torch.from_numpy(batches[which]))
        say(f"graph ({size}): replay {rep} on batch {which}")
        g.replay()
        torch.cuda.synchronize()
        for got, w in zip(ys, want[which]):
            assert torch.equal(got, w), (rep, which)
