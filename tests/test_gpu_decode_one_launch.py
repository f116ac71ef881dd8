"""The one-launch ("chained") form of the decode call: shrink units first in the grid, expand units after them, the
sums handed over inside the launch through arrival counters in the work records (mlora_bgmv_multi with a workspace on
batches of about one round of workgroups; replaces punica.ops.add_lora_bgmv, lora_gpu.py:138,150,162).

Checked here, through the C ABI: against the oracle and against an fp32 evaluation on the device (rtol 1e-2 / atol
1e-3); that it agrees with the two-launch form; that the records are left exactly as the gather wrote them; that
repeated calls through one plan and one workspace never see an earlier call's sums; that it still gives the right
result when every wait is made to time out (each expand unit then computes the sums itself) and when each workgroup
has to take several units (a small grid cap); and that a HIP graph of it replays to the eager bits.
"""
import numpy as np
import pytest
import torch

from gpu_common import ATOL, RTOL, assert_close_bits, oracle_apply, say, upload_pool
from helpers import BF16, FP16, PagedPool, bits_of, bits_to_torch, torch_to_bits
from mlora import _ext, bgmv, plan_decode, workloads

pytestmark = pytest.mark.gpu


@pytest.fixture
def options():
    """Process-wide options are put back after every test."""
    lib = _ext.lib()

    def set_(**kw):
        for k, v in kw.items():
            _ext.check(lib.mlora_set_option(getattr(_ext, "OPT_DECODE_" + k.upper()), v))
    yield set_
    set_(one_launch=1, spin_limit=1 << 20, grid_cap=2048)


def _zipf(rng, T, N, alpha):
    p = np.arange(1, N + 1, dtype=np.float64) ** -alpha
    return rng.permutation(N)[rng.choice(N, size=T, p=p / p.sum())].astype(np.int32)


def _device_reference(pool, layer, names, xs, y0, tok_np):
    want = [y.float().clone() for y in y0]
    for a in np.unique(tok_np[tok_np >= 0]):
        idx = torch.from_numpy(np.nonzero(tok_np == a)[0]).cuda()
        rows = pool.rows_of(int(a))
        for i, p in enumerate(names):
            A = pool.a_rows[p][layer][rows].float()
            B = pool.b_rows[p][layer][rows].float()
            want[i][idx] += float(pool.h_scaling[a]) * ((xs[i][idx].float() @ A.t()) @ B)
    return want


def _close(got, want):
    err = (got.float() - want).abs()
    return bool((err <= ATOL + RTOL * want.abs()).all()), float(err.max())


CASES = [
    # name, T, ranks (None = mixed), projections, alpha, group
    ("config 2", 256, [16] * 64, ["q", "k", "v", "o"], 1.0, 4),
    ("config 3", 128, None, ["q", "k", "v", "o", "gate", "up", "down"], 1.2, 4),
    ("rank 32, 96 tokens, groups of 2", 96, [32] * 40, ["q", "gate", "down"], 1.0, 2),
    ("mixed ranks, groups of 1, tokens without adapter", 70, None, ["q", "down"], 0.8, 1),
]


@pytest.mark.parametrize("name,T,ranks,names,alpha,group", CASES, ids=[c[0] for c in CASES])
@pytest.mark.parametrize("variant", ["default", "timeouts", "small grid"])
def test_one_launch_form(name, T, ranks, names, alpha, group, variant, options):
    rng = np.random.default_rng(sum(map(ord, name)))
    N = 128 if ranks is None else len(ranks)
    if ranks is None:
        ranks = rng.choice([8, 16, 24, 32, 64], N).astype(np.int32)
    shapes = {p: workloads.LLAMA7B_ALL[p] for p in names}
    wl = workloads.make_decode("one-launch", shapes, 1, T, N, ranks, alpha, seed=int(rng.integers(1 << 30)), device="cuda")
    pool, tok_np = wl.pool, wl.tok_adapter.copy()
    if "without adapter" in name:
        tok_np[rng.random(T) < 0.1] = -1
    tok = torch.from_numpy(tok_np).cuda()
    gen = torch.Generator(device="cuda").manual_seed(3)
    plan = plan_decode(tok, pool, group=group)
    torch.cuda.synchronize()
    records = plan.work.clone()
    if variant == "timeouts":
        options(spin_limit=0)                  # no poll ever succeeds: every expand unit computes the sums itself
    elif variant == "small grid":
        options(grid_cap=64)                   # 64 workgroups per part: each takes many units
    for rep in range(3):                       # the same plan and workspace, new inputs every time
        xs = [torch.randn(T, shapes[p][0], device="cuda", generator=gen).half() for p in names]
        y0 = [torch.randn(T, shapes[p][1], device="cuda", generator=gen).half() for p in names]
        for accumulate in (True, False):
            ys = [y.clone() if accumulate else torch.full_like(y, float("nan")) for y in y0]
            say(f"one launch: {name}, {variant}, call {rep}, accumulate={accumulate}")
            bgmv(ys, xs, pool, 0, names, tok, plan=plan, accumulate=accumulate, fused=False)
            torch.cuda.synchronize()
            base = y0 if accumulate else [torch.zeros_like(y) for y in y0]
            want = _device_reference(pool, 0, names, xs, base, tok_np)
            for i, p in enumerate(names):
                ok, worst = _close(ys[i], want[i])
                assert ok, (p, rep, accumulate, worst)
                if accumulate:
                    none = torch.from_numpy(np.nonzero(tok_np < 0)[0]).cuda()
                    assert torch.equal(ys[i][none], y0[i][none])
            assert torch.equal(plan.work, records), "the call left its counters in the work records"
    # ... and the two-launch form on the last inputs agrees
    options(one_launch=0)
    y2 = [y.clone() for y in y0]
    y1 = [y.clone() for y in y0]
    say(f"two launches: {name}")
    bgmv(y2, xs, pool, 0, names, tok, plan=plan, fused=False)
    options(one_launch=1)
    bgmv(y1, xs, pool, 0, names, tok, plan=plan, fused=False)
    torch.cuda.synchronize()
    for a, b in zip(y1, y2):
        assert torch.allclose(a.float(), b.float(), rtol=RTOL, atol=ATOL)


def test_one_launch_against_the_oracle_and_bit_exact_on_integers(options):
    rng = np.random.default_rng(91)
    ranks = [8, 16, 3, 64, 5, 32, 24]
    for integer in (False, True):
        pp = PagedPool(rng, ranks, hin=1032, hout=776, page_rows=8, dtype=BF16 if not integer else FP16, integer=integer)
        if integer:
            pp.scaling[:] = [1, 2, 0.5, -1, 4, 0.25, 1]
        T = 90
        tok = rng.integers(-1, len(ranks), T).astype(np.int32)
        if integer:
            x = bits_of((rng.integers(-2, 3, (T, 1032)) * (rng.random((T, 1032)) < 0.04)).astype(np.float32), pp.dtype)
            y0 = bits_of(rng.integers(-8, 9, (T, 776)).astype(np.float32), pp.dtype)
        else:
            x = bits_of(rng.standard_normal((T, 1032)).astype(np.float32), pp.dtype)
            y0 = bits_of(rng.standard_normal((T, 776)).astype(np.float32), pp.dtype)
        want = oracle_apply(pp, x, tok, y0)
        pool = upload_pool(pp)
        t = torch.from_numpy(tok).cuda()
        for group in (1, 2, 4):
            for spin in (1 << 20, 0):
                options(spin_limit=spin)
                plan = plan_decode(t, pool, group=group)
                y = bits_to_torch(y0, pp.dtype, "cuda")
                say(f"one launch vs oracle: integer={integer} group={group} spin_limit={spin}")
                bgmv([y], [bits_to_torch(x, pp.dtype, "cuda")], pool, 0, ["p"], t, plan=plan, fused=False)
                torch.cuda.synchronize()
                if integer:
                    assert np.array_equal(torch_to_bits(y), want), (group, spin)
                else:
                    assert_close_bits(torch_to_bits(y), want, pp.dtype, f"group {group} spin {spin}")


def test_one_launch_graph_replays(options):
    """Three replays with eager work and synchronisations between them, every replay against the eager result."""
    rng = np.random.default_rng(17)
    names = ["q", "k", "v", "o"]
    shapes = {p: workloads.LLAMA7B_ATTN[p] for p in names}
    T = 200
    wl = workloads.make_decode("one-launch graph", shapes, 2, T, 48, [16], 1.0, seed=18, device="cuda")
    pool = wl.pool
    tok = torch.from_numpy(wl.tok_adapter).cuda()
    gen = torch.Generator(device="cuda").manual_seed(4)
    xs = [[torch.randn(T, 4096, device="cuda", generator=gen).half() for _ in names] for _ in range(2)]
    y0 = [[torch.randn(T, 4096, device="cuda", generator=gen).half() for _ in names] for _ in range(2)]
    ys = [[y.clone() for y in layer] for layer in y0]
    plan = plan_decode(tok, pool, group=4)

    def step():
        plan_decode(tok, pool, group=4, out=plan)
        for l in range(2):
            bgmv(ys[l], xs[l], pool, l, names, tok, plan=plan, fused=False)

    say("one launch: eager step")
    step()
    torch.cuda.synchronize()
    eager = [[y.clone() for y in layer] for layer in ys]
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    for rep in range(3):
        for l in range(2):
            for y, y_init in zip(ys[l], y0[l]):
                y.copy_(y_init)
        scratch = torch.randn(1 << 20, device="cuda").sum()          # eager work between the replays
        torch.cuda.synchronize()
        say(f"one launch: graph replay {rep}")
        g.replay()
        torch.cuda.synchronize()
        for l in range(2):
            for a, b in zip(ys[l], eager[l]):
                assert torch.equal(a, b), (rep, l)
        del scratch
