"""The mixed step of config 5 on a multi-layer pool at its real row count: per layer one decode call
(`bgmv`, two launches) and one prefill call (`sgmv_multi`, three launches) that share the pool and the plans,
side by side on two streams and joined before the next layer, as `bench.py --workload c5` runs it, eagerly and
replayed from a HIP graph.

Every layer is checked against a plain fp32 evaluation on the device (adapter by adapter, over the rows the pool's
page table names); the first and the last layer are also checked against the CPU oracle on a sample of decode and
prefill tokens.  Tolerance as everywhere: rtol 1e-2 / atol 1e-3.  Projections q, gate and down (one of each
shape) keep the pool at 20 GB.
"""
import numpy as np
import pytest
import torch

from gpu_common import ATOL, RTOL, say
from mlora import SideStream, bgmv, plan_decode, plan_prefill, sgmv_multi, side_by_side, workloads
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

LAYERS = 8
N_ADAPTERS, RANK = 1000, 32
T_DEC, N_SEG, SEG_LEN = 512, 8, 512
SHAPES = {p: workloads.LLAMA7B_ALL[p] for p in ("q", "gate", "down")}


def _device_reference(pool, layer, names, xs, y0, ids_per_adapter):
    """fp32 on the device: y0 + s_a (x A_a^T) B_a for the tokens of every adapter."""
    want = {p: y0[p].float().clone() for p in names}
    for a, idx in ids_per_adapter:
        rows = pool.rows_of(int(a))
        for p in names:
            A = pool.a_rows[p][layer][rows].float()
            B = pool.b_rows[p][layer][rows].float()
            want[p][idx] += float(pool.h_scaling[a]) * ((xs[p][idx].float() @ A.t()) @ B)
    return want


def _oracle_on_sample(pool, layer, p, x, y0, got, tok_adapter, sample):
    """The CPU oracle on the sampled tokens: their adapters' rows are copied into a small dense pool."""
    ads = np.unique(tok_adapter[sample])
    remap = {int(a): i for i, a in enumerate(ads)}
    pages_per = RANK // pool.page_rows
    a_rows = torch.cat([pool.a_rows[p][layer][pool.rows_of(int(a))] for a in ads]).cpu().numpy().view(np.uint16)
    b_rows = torch.cat([pool.b_rows[p][layer][pool.rows_of(int(a))] for a in ads]).cpu().numpy().view(np.uint16)
    tbl = np.arange(len(ads) * pages_per, dtype=np.int32).reshape(len(ads), pages_per)
    tok = np.array([remap[int(tok_adapter[t])] for t in sample], np.int32)
    idx = torch.from_numpy(np.asarray(sample)).cuda()
    want = orc.lora_apply_paged(x[idx].cpu().numpy().view(np.uint16), a_rows, b_rows, tok, tbl, tbl,
                                np.full(len(ads), RANK, np.int32), pool.h_scaling[ads].astype(np.float32), pool.page_rows,
                                orc.FP16, y0=y0[idx].cpu().numpy().view(np.uint16)).view(np.float16).astype(np.float32)
    have = got[idx].float().cpu().numpy()
    err = np.abs(have - want)
    assert np.all(err <= ATOL + RTOL * np.abs(want)), (p, layer, float(err.max()))


def test_mixed_step_config5_rows_eight_layers():
    names = list(SHAPES)
    wl = workloads.make_decode("c5-mixed", SHAPES, LAYERS, T_DEC, N_ADAPTERS, [RANK], 1.1, seed=1005, device="cuda")
    pool = wl.pool
    rng = np.random.default_rng(77)
    tok_np = wl.tok_adapter
    tok = torch.from_numpy(tok_np).cuda()
    seg_adapter = workloads.zipf_adapters(rng, N_SEG, N_ADAPTERS, 1.1)
    Tp = N_SEG * SEG_LEN
    ss = torch.arange(0, Tp, SEG_LEN, dtype=torch.int32, device="cuda")
    sl = torch.full((N_SEG,), SEG_LEN, dtype=torch.int32, device="cuda")
    sa = torch.from_numpy(seg_adapter).cuda()
    pre_tok_adapter = np.repeat(seg_adapter, SEG_LEN)
    gen = torch.Generator(device="cuda").manual_seed(9)
    # every layer has its own activations and outputs, as in the benchmark's decode half
    dx = [{p: torch.randn(T_DEC, SHAPES[p][0], device="cuda", generator=gen).half() for p in names} for _ in range(LAYERS)]
    dy0 = [{p: torch.randn(T_DEC, SHAPES[p][1], device="cuda", generator=gen).half() for p in names} for _ in range(LAYERS)]
    px = {p: torch.randn(Tp, SHAPES[p][0], device="cuda", generator=gen).half() for p in names}
    py0 = {p: torch.randn(Tp, SHAPES[p][1], device="cuda", generator=gen).half() for p in names}
    dy = [{p: dy0[l][p].clone() for p in names} for l in range(LAYERS)]
    py = [{p: py0[p].clone() for p in names} for _ in range(LAYERS)]

    plan = plan_decode(tok, pool, group=4)
    pplan = plan_prefill(ss, sl, sa, Tp, pool, n_proj=len(names))
    side = SideStream("cuda")

    def step():
        for l in range(LAYERS):
            side_by_side(side,
                         lambda l=l: sgmv_multi([py[l][p] for p in names], [px[p] for p in names], pool, l, names, pplan),
                         lambda l=l: bgmv([dy[l][p] for p in names], [dx[l][p] for p in names], pool, l, names, tok,
                                          plan=plan, fused=False))

    say(f"mixed step, {LAYERS} layers x {len(names)} projections, {N_ADAPTERS} rank-{RANK} adapters, "
        f"{T_DEC} decode + {Tp} prefill tokens, two streams, eager")
    step()
    torch.cuda.synchronize()

    dec_groups = [(a, torch.from_numpy(np.nonzero(tok_np == a)[0]).cuda()) for a in np.unique(tok_np)]
    pre_groups = [(a, torch.from_numpy(np.nonzero(pre_tok_adapter == a)[0]).cuda()) for a in np.unique(seg_adapter)]
    dec_sample = rng.choice(T_DEC, 24, replace=False)
    pre_sample = np.concatenate([[0, SEG_LEN - 1, SEG_LEN, Tp - 1], rng.choice(Tp, 20, replace=False)])
    eager = []
    for l in range(LAYERS):
        want_d = _device_reference(pool, l, names, dx[l], dy0[l], dec_groups)
        want_p = _device_reference(pool, l, names, px, py0, pre_groups)
        for p in names:
            assert torch.allclose(dy[l][p].float(), want_d[p], rtol=RTOL, atol=ATOL), ("decode", l, p)
            assert torch.allclose(py[l][p].float(), want_p[p], rtol=RTOL, atol=ATOL), ("prefill", l, p)
        if l in (0, LAYERS - 1):
            for p in names:
                _oracle_on_sample(pool, l, p, dx[l][p], dy0[l][p], dy[l][p], tok_np, dec_sample)
                _oracle_on_sample(pool, l, p, px[p], py0[p], py[l][p], pre_tok_adapter, pre_sample)
        eager.append(({p: dy[l][p].clone() for p in names}, {p: py[l][p].clone() for p in names}))

    # the same step replayed from a HIP graph gives the same bits as the eager run
    for l in range(LAYERS):
        for p in names:
            dy[l][p].copy_(dy0[l][p])
            py[l][p].copy_(py0[p])
    torch.cuda.synchronize()
    say("mixed step captured into a HIP graph and replayed")
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    for l in range(LAYERS):                      # the capture pass ran nothing: outputs still hold y0
        for p in names:
            assert torch.equal(dy[l][p], dy0[l][p])
    g.replay()
    torch.cuda.synchronize()
    for l in range(LAYERS):
        for p in names:
            assert torch.equal(dy[l][p], eager[l][0][p]), ("decode replay", l, p)
            assert torch.equal(py[l][p], eager[l][1][p]), ("prefill replay", l, p)
