"""GPU parity: BGMV decode through the C ABI, fused launch and shrink + expand pair, against the
fp32-accumulated oracle (rtol 1e-2 / atol 1e-3), on seeded inputs, plus size-independent
properties at full size."""
import zlib

import numpy as np
import pytest
import torch

from gpu_common import (ATOL, RTOL, assert_close_bits, oracle_apply, say, tdtype, upload_pool)
from helpers import BF16, FP16, PagedPool, bits_of, bits_to_torch, f32_of, torch_to_bits
from mlora import bgmv, lora_apply, plan_decode

pytestmark = pytest.mark.gpu


def _zipf(rng, T, N, alpha):
    p = np.arange(1, N + 1, dtype=np.float64) ** -alpha
    return rng.permutation(N)[rng.choice(N, size=T, p=p / p.sum())].astype(np.int32)


def _run(pp, x_bits, tok, y0_bits, group, accumulate=True, fused=None):
    pool = upload_pool(pp)
    x = bits_to_torch(x_bits, pp.dtype, "cuda")
    y = bits_to_torch(y0_bits, pp.dtype, "cuda") if y0_bits is not None else \
        torch.full((len(tok), pp.hout), float("nan"), dtype=tdtype(pp.dtype), device="cuda")
    t = torch.from_numpy(tok).cuda()
    plan = plan_decode(t, pool, group=group) if group > 0 else None
    bgmv([y], [x], pool, 0, ["p"], t, plan=plan, accumulate=accumulate, fused=fused)
    torch.cuda.synchronize()
    return torch_to_bits(y)


# launch forms: (group, fused); group 0 = no plan, one token per work item
FORMS = [(0, True), (1, True), (2, True), (4, True), (1, False), (2, False), (4, False)]


CASES = [
    # name, T, ranks, hin, hout, alpha, dtype
    ("C1 q_proj T=32 8xr16", 32, [16] * 8, 4096, 4096, 0.0, FP16),
    ("C2 q_proj T=256 64xr16 zipf1.0", 256, [16] * 64, 4096, 4096, 1.0, FP16),
    ("C2 bf16", 256, [16] * 64, 4096, 4096, 1.0, BF16),
    ("C3 hetero 4096x4096", 128, None, 4096, 4096, 1.2, FP16),
    ("C3 hetero gate 4096x11008", 128, None, 4096, 11008, 1.2, FP16),
    ("C3 hetero down 11008x4096", 128, None, 11008, 4096, 1.2, FP16),
    ("C5 slice T=512 r32", 512, [32] * 200, 4096, 4096, 1.1, FP16),
    ("odd widths 200x72", 19, [8, 24, 5, 64, 1], 200, 72, 0.5, BF16),
]


_CASE_CACHE = {}


def _case(name):
    """Seeded inputs and oracle outputs of one case (computed once, shared by the launch variants)."""
    if name not in _CASE_CACHE:
        _, T, ranks, hin, hout, alpha, dtype = next(c for c in CASES if c[0] == name)
        rng = np.random.default_rng(zlib.crc32(name.encode()))
        if ranks is None:
            ranks = rng.choice([8, 16, 32, 64], 128)
        N = len(ranks)
        pp = PagedPool(rng, ranks, hin, hout, page_rows=8, dtype=dtype)
        tok = _zipf(rng, T, N, alpha) if alpha > 0 else rng.integers(0, N, T).astype(np.int32)
        x = bits_of(rng.standard_normal((T, hin)).astype(np.float32), dtype)
        y0 = bits_of(rng.standard_normal((T, hout)).astype(np.float32), dtype)
        _CASE_CACHE[name] = (pp, tok, x, y0, oracle_apply(pp, x, tok, y0), oracle_apply(pp, x, tok, None))
    return _CASE_CACHE[name]


@pytest.mark.parametrize("name", [c[0] for c in CASES])
@pytest.mark.parametrize("group,fused", FORMS)
def test_bgmv_vs_oracle(name, group, fused):
    dtype = next(c for c in CASES if c[0] == name)[6]
    pp, tok, x, y0, want, want_d = _case(name)
    say(f"bgmv {name} group={group} fused={fused} accumulate")
    got = _run(pp, x, tok, y0, group, fused=fused)
    assert_close_bits(got, want, dtype, name)
    # the delta alone must also meet the tolerance (y = delta form, reference's zeros+bgmv at lora_gpu.py:137-138)
    say(f"bgmv {name} group={group} fused={fused} delta")
    got_d = _run(pp, x, tok, None, group, accumulate=False, fused=fused)
    assert_close_bits(got_d, want_d, dtype, name + " delta")


@pytest.mark.parametrize("group,fused", [(0, True), (2, True), (8, True), (1, False), (2, False), (8, False)])
def test_bgmv_integer_inputs_bit_exact(group, fused):
    """Integer-valued inputs make every fp32 operation exact: the kernel must match bit for bit."""
    rng = np.random.default_rng(41)
    ranks = [8, 16, 3, 1, 5, 32]
    pp = PagedPool(rng, ranks, hin=512, hout=256, page_rows=8, dtype=FP16, integer=True)
    pp.scaling[:] = [1, 2, 0.5, -1, 4, 0.25]
    T = 61
    tok = rng.integers(-1, len(ranks), T).astype(np.int32)
    # sparse integer activations keep |sums| < 2048 (exact in fp16)
    xi = (rng.integers(-2, 3, (T, 512)) * (rng.random((T, 512)) < 0.06)).astype(np.float32)
    y0 = bits_of(rng.integers(-8, 9, (T, 256)).astype(np.float32), FP16)
    x = bits_of(xi, FP16)
    want = oracle_apply(pp, x, tok, y0)
    assert np.abs(f32_of(want, FP16)).max() < 2048
    say(f"bgmv integer-valued inputs group={group} fused={fused}")
    got = _run(pp, x, tok, y0, group, fused=fused)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("T,want_group,want_fused", [(48, 1, True), (100, 2, True), (300, 4, False)])
def test_bgmv_default_form_by_batch_size(T, want_group, want_fused):
    """Without `group` and `fused` the host layer picks them from the batch size; the result is the
    explicitly requested form's, bit for bit, and meets the oracle's tolerance."""
    from mlora import ops
    rng = np.random.default_rng(300 + T)
    pp = PagedPool(rng, [16] * 12, 1024, 1024, page_rows=8, dtype=FP16)
    tok = rng.integers(0, 12, T).astype(np.int32)
    x = bits_of(rng.standard_normal((T, 1024)).astype(np.float32), FP16)
    y0 = bits_of(rng.standard_normal((T, 1024)).astype(np.float32), FP16)
    pool = upload_pool(pp)
    t = torch.from_numpy(tok).cuda()
    plan = plan_decode(t, pool)
    assert plan.group == want_group and ops.decode_fused(T, plan.group, 1, pool.n_slots) == want_fused
    say(f"bgmv default form T={T}")
    y = bits_to_torch(y0, FP16, "cuda")
    bgmv([y], [bits_to_torch(x, FP16, "cuda")], pool, 0, ["p"], t, plan=plan)
    torch.cuda.synchronize()
    got = torch_to_bits(y)
    assert_close_bits(got, oracle_apply(pp, x, tok, y0), FP16, f"default form T={T}")
    assert np.array_equal(got, _run(pp, x, tok, y0, want_group, fused=want_fused))


def test_bgmv_tokens_without_adapter_and_rank_tails():
    rng = np.random.default_rng(42)
    pp = PagedPool(rng, [7, 9, 33, 64, 2], 1024, 1024, page_rows=8, dtype=FP16)
    T = 40
    tok = rng.integers(-1, 5, T).astype(np.int32)
    tok[:3] = -1
    x = bits_of(rng.standard_normal((T, 1024)).astype(np.float32), FP16)
    y0 = bits_of(rng.standard_normal((T, 1024)).astype(np.float32), FP16)
    for group, fused in ((0, True), (4, True), (4, False), (2, False)):
        say(f"bgmv no-adapter tokens group={group} fused={fused}")
        got = _run(pp, x, tok, y0, group, fused=fused)
        assert np.array_equal(got[tok < 0], y0[tok < 0])          # untouched, bit for bit
        assert_close_bits(got, oracle_apply(pp, x, tok, y0), FP16)
        got_d = _run(pp, x, tok, None, group, accumulate=False, fused=fused)
        assert np.all(got_d[tok < 0] == 0)                        # y = delta defines those rows as zero
        assert_close_bits(got_d, oracle_apply(pp, x, tok, None), FP16)


def test_bgmv_ids_below_minus_one_and_beyond_the_pool_mean_no_adapter():
    """An int32 id < -1 or >= n_adapters is "no adapter" in every launch form: the row is kept when
    accumulating and is zeros in y = delta mode (a caller may hand over torch.empty memory)."""
    rng = np.random.default_rng(43)
    N = 5
    pp = PagedPool(rng, [8, 16, 4, 32, 2], 512, 384, page_rows=8, dtype=FP16)
    T = 37
    tok = rng.integers(0, N, T).astype(np.int32)
    tok[[1, 7, 20]] = -2
    tok[[3, 8]] = N + 3
    tok[11] = -1
    tok[30] = np.iinfo(np.int32).max
    tok[31] = np.iinfo(np.int32).min
    none = (tok < 0) | (tok >= N)
    tok_orc = np.where(none, -1, tok).astype(np.int32)      # the oracle's spelling of "no adapter"
    x = bits_of(rng.standard_normal((T, 512)).astype(np.float32), FP16)
    y0 = bits_of(rng.standard_normal((T, 384)).astype(np.float32), FP16)
    want, want_d = oracle_apply(pp, x, tok_orc, y0), oracle_apply(pp, x, tok_orc, None)
    for group, fused in ((0, True), (1, True), (4, True), (4, False)):
        say(f"bgmv out-of-range ids group={group} fused={fused}")
        got = _run(pp, x, tok, y0, group, fused=fused)
        assert np.array_equal(got[none], y0[none])
        assert_close_bits(got, want, FP16)
        got_d = _run(pp, x, tok, None, group, accumulate=False, fused=fused)      # y starts as NaN
        assert np.all(got_d[none] == 0)
        assert_close_bits(got_d, want_d, FP16)


def test_bgmv_multi_projection_one_launch():
    """q/k/v share x, o has its own input: one launch, four slabs, each checked against the oracle."""
    rng = np.random.default_rng(43)
    T, N, H = 96, 24, 1024
    ranks = rng.choice([8, 16, 32], N)
    pps = {p: PagedPool(np.random.default_rng(50), ranks, H, H, page_rows=8, dtype=FP16) for p in "qkvo"}
    for i, p in enumerate("qkvo"):      # same page table, different weights per projection
        r2 = np.random.default_rng(60 + i)
        pps[p].a_rows = bits_of((r2.standard_normal(pps[p].a_rows.shape) * 0.02).astype(np.float32), FP16)
        pps[p].b_rows = bits_of((r2.standard_normal(pps[p].b_rows.shape) * 0.02).astype(np.float32), FP16)
    pool = upload_pool(pps["q"], projections={p: (H, H) for p in "qkvo"})
    for p in "qkvo":
        pool.a_rows[p][0].copy_(bits_to_torch(pps[p].a_rows, FP16))
        pool.b_rows[p][0].copy_(bits_to_torch(pps[p].b_rows, FP16))
    tok = _zipf(rng, T, N, 1.0)
    x_qkv = bits_of(rng.standard_normal((T, H)).astype(np.float32), FP16)
    x_o = bits_of(rng.standard_normal((T, H)).astype(np.float32), FP16)
    y0 = {p: bits_of(rng.standard_normal((T, H)).astype(np.float32), FP16) for p in "qkvo"}
    t = torch.from_numpy(tok).cuda()
    xs = {p: bits_to_torch(x_o if p == "o" else x_qkv, FP16, "cuda") for p in "qkvo"}
    ys = {p: bits_to_torch(y0[p], FP16, "cuda") for p in "qkvo"}
    plan = plan_decode(t, pool, group=4)
    for fused in (True, False):
        ys = {p: bits_to_torch(y0[p], FP16, "cuda") for p in "qkvo"}
        say(f"bgmv 4 projections in one call fused={fused}")
        bgmv([ys[p] for p in "qkvo"], [xs[p] for p in "qkvo"], pool, 0, list("qkvo"), t, plan=plan, fused=fused)
        torch.cuda.synchronize()
        for p in "qkvo":
            want = oracle_apply(pps[p], x_o if p == "o" else x_qkv, tok, y0[p])
            assert_close_bits(torch_to_bits(ys[p]), want, FP16, f"projection {p}")


def test_bgmv_full_size_properties():
    """Config-2 size, no oracle: permutation equivariance, page-placement invariance, grouped == ungrouped
    within tolerance, linearity of the delta, and lora_apply == bgmv."""
    rng = np.random.default_rng(44)
    T, N, H = 256, 64, 4096
    pp = PagedPool(rng, [16] * N, H, H, page_rows=8, dtype=FP16)
    pool = upload_pool(pp)
    tok = _zipf(rng, T, N, 1.0)
    x = torch.randn(T, H, device="cuda", dtype=torch.float16)
    y0 = torch.randn(T, H, device="cuda", dtype=torch.float16)
    t = torch.from_numpy(tok).cuda()

    def run(xx, tt, yy0, group, fused=True):
        y = yy0.clone()
        plan = plan_decode(tt, pool, group=group) if group else None
        bgmv([y], [xx], pool, 0, ["p"], tt, plan=plan, fused=fused)
        return y

    say("bgmv full-size: direct vs grouped")
    y_direct = run(x, t, y0, 0)
    y_g4 = run(x, t, y0, 4)
    y_g8 = run(x, t, y0, 8)
    y_s2, y_s4, y_s8 = (run(x, t, y0, g, fused=False) for g in (2, 4, 8))
    torch.cuda.synchronize()
    for other in (y_g4, y_g8, y_s4):
        assert torch.allclose(other.float(), y_direct.float(), rtol=RTOL, atol=ATOL)
    # a token's result does not depend on which other tokens share its work item: within one launch
    # form the summation order is fixed, so the results agree bit for bit
    assert torch.equal(y_g4, y_direct) and torch.equal(y_g8, y_direct)
    assert torch.equal(y_s2, y_s4) and torch.equal(y_s8, y_s4)
    say("bgmv full-size: token permutation")
    perm = torch.randperm(T, device="cuda")
    y_perm = run(x[perm].contiguous(), t[perm].contiguous(), y0[perm].contiguous(), 4)
    assert torch.equal(y_perm, y_g4[perm])
    y_perm = run(x[perm].contiguous(), t[perm].contiguous(), y0[perm].contiguous(), 4, fused=False)
    assert torch.equal(y_perm, y_s4[perm])
    say("bgmv full-size: lora_apply")
    y_api = lora_apply(y0.clone(), x, t, pool, 0, "p")
    torch.cuda.synchronize()
    assert torch.equal(y_api, y_direct)
    say("bgmv full-size: page placement")
    pp2 = PagedPool(np.random.default_rng(7), [16] * N, H, H, page_rows=8, dtype=FP16, extra_pages=9)
    for i in range(N):
        pp2.a_rows[pp2.rows(i)] = pp.a_rows[pp.rows(i)]
        pp2.b_rows[pp2.rows(i)] = pp.b_rows[pp.rows(i)]
    pool2 = upload_pool(pp2)
    y2 = y0.clone()
    bgmv([y2], [x], pool2, 0, ["p"], t, plan=plan_decode(t, pool2, group=4), fused=True)
    y3 = y0.clone()
    bgmv([y3], [x], pool2, 0, ["p"], t, plan=plan_decode(t, pool2, group=4), fused=False)
    torch.cuda.synchronize()
    assert torch.equal(y2, y_g4) and torch.equal(y3, y_s4)
    say("bgmv full-size: linearity of the delta")
    d1 = torch.zeros_like(y0)
    d2 = torch.zeros_like(y0)
    bgmv([d1], [x], pool, 0, ["p"], t, accumulate=False)
    bgmv([d2], [(2 * x).contiguous()], pool, 0, ["p"], t, accumulate=False)
    torch.cuda.synchronize()
    normal = d1.abs() >= 2.0 ** -13
    assert torch.equal(d2[normal], 2 * d1[normal])


@pytest.mark.parametrize("fused", [True, False])
def test_bgmv_projections_of_different_widths_in_one_call(fused):
    """Seven projections with the widths of a (scaled-down) MLP + attention block, ragged against the
    column slices of the two-launch form: 2056 columns = one slice plus one 16-byte chunk."""
    rng = np.random.default_rng(45)
    shapes = {"q": (512, 512), "k": (512, 128), "v": (512, 128), "o": (512, 512),
              "gate": (512, 2056), "up": (512, 2056), "down": (2056, 512)}
    T, N = 37, 9
    ranks = rng.choice([8, 16, 32, 64, 5], N)
    pps = {p: PagedPool(np.random.default_rng(51), ranks, hin, hout, page_rows=8, dtype=BF16) for p, (hin, hout) in shapes.items()}
    for i, p in enumerate(shapes):
        r2 = np.random.default_rng(70 + i)
        pps[p].a_rows = bits_of((r2.standard_normal(pps[p].a_rows.shape) * 0.02).astype(np.float32), BF16)
        pps[p].b_rows = bits_of((r2.standard_normal(pps[p].b_rows.shape) * 0.02).astype(np.float32), BF16)
    pool = upload_pool(pps["q"], projections=shapes)
    for p in shapes:
        pool.a_rows[p][0].copy_(bits_to_torch(pps[p].a_rows, BF16))
        pool.b_rows[p][0].copy_(bits_to_torch(pps[p].b_rows, BF16))
    tok = rng.integers(-1, N, T).astype(np.int32)
    xin = {512: bits_of(rng.standard_normal((T, 512)).astype(np.float32), BF16),
           2056: bits_of(rng.standard_normal((T, 2056)).astype(np.float32), BF16)}
    y0 = {p: bits_of(rng.standard_normal((T, shapes[p][1])).astype(np.float32), BF16) for p in shapes}
    t = torch.from_numpy(tok).cuda()
    xs = {h: bits_to_torch(v, BF16, "cuda") for h, v in xin.items()}
    ys = {p: bits_to_torch(y0[p], BF16, "cuda") for p in shapes}
    names = list(shapes)
    say(f"bgmv 7 projections of different widths fused={fused}")
    bgmv([ys[p] for p in names], [xs[shapes[p][0]] for p in names], pool, 0, names, t,
         plan=plan_decode(t, pool, group=2), fused=fused)
    torch.cuda.synchronize()
    for p in names:
        want = oracle_apply(pps[p], xin[shapes[p][0]], tok, y0[p])
        assert_close_bits(torch_to_bits(ys[p]), want, BF16, f"projection {p}")


def test_bgmv_config5_one_layer_full_pool():
    """Config 5 at its real pool size for one layer: 1000 rank-32 adapters (32000 rank rows per slab, 5 GB of
    slabs), 512 decode tokens Zipf(1.1), all seven Llama-7B projections in one call.  Too large for the
    CPU oracle in a test, so the check is a plain fp32 evaluation on the device, adapter by adapter, of
    the rows the pool's own page table names (tolerance as everywhere: rtol 1e-2 / atol 1e-3), for both
    launch forms, plus agreement of the prefill kernels with the decode kernels on the same tokens."""
    from mlora import plan_prefill, sgmv_multi, workloads
    wl = workloads.make_decode("c5-layer", workloads.LLAMA7B_ALL, 1, 512, 1000, [32], 1.1, seed=1005, device="cuda")
    pool = wl.pool
    names = list(workloads.LLAMA7B_ALL)
    T = 512
    tok = torch.from_numpy(wl.tok_adapter).cuda()
    gen = torch.Generator(device="cuda").manual_seed(5)
    xs = {h: torch.randn(T, h, device="cuda", generator=gen).half() for h in (4096, 11008)}
    y0 = {p: torch.randn(T, workloads.LLAMA7B_ALL[p][1], device="cuda", generator=gen).half() for p in names}
    want = {p: y0[p].float().clone() for p in names}
    for a in np.unique(wl.tok_adapter):
        idx = torch.from_numpy(np.nonzero(wl.tok_adapter == a)[0]).cuda()
        rows = pool.rows_of(int(a))
        for p in names:
            hin, _ = workloads.LLAMA7B_ALL[p]
            A = pool.a_rows[p][0][rows].float()                 # [r, hin]
            B = pool.b_rows[p][0][rows].float()                 # [r, hout]
            want[p][idx] += float(pool.h_scaling[a]) * ((xs[hin][idx].float() @ A.t()) @ B)
    plan = plan_decode(tok, pool, group=4)
    got = {}
    for fused in (False, True):
        ys = {p: y0[p].clone() for p in names}
        say(f"bgmv config-5 layer, 1000 adapters, 7 projections, fused={fused}")
        bgmv([ys[p] for p in names], [xs[workloads.LLAMA7B_ALL[p][0]] for p in names], pool, 0, names, tok, plan=plan,
             fused=fused)
        torch.cuda.synchronize()
        for p in names:
            assert torch.allclose(ys[p].float(), want[p], rtol=RTOL, atol=ATOL), (p, fused)
        got[fused] = ys
    # the same tokens as a prefill batch: sorted by adapter they form segments
    order = np.argsort(wl.tok_adapter, kind="stable")
    sorted_ad = wl.tok_adapter[order]
    starts = np.flatnonzero(np.r_[True, sorted_ad[1:] != sorted_ad[:-1]]).astype(np.int32)
    lens = np.diff(np.r_[starts, T]).astype(np.int32)
    o = torch.from_numpy(order).cuda()
    pplan = plan_prefill(torch.from_numpy(starts).cuda(), torch.from_numpy(lens).cuda(),
                         torch.from_numpy(sorted_ad[starts].astype(np.int32)).cuda(), T, pool, n_proj=len(names))
    ys = {p: y0[p][o].contiguous() for p in names}
    xo = {h: xs[h][o].contiguous() for h in xs}
    say("sgmv_multi on the same tokens grouped into segments")
    sgmv_multi([ys[p] for p in names], [xo[workloads.LLAMA7B_ALL[p][0]] for p in names], pool, 0, names, pplan)
    torch.cuda.synchronize()
    for p in names:
        assert torch.allclose(ys[p].float(), want[p][o], rtol=RTOL, atol=ATOL), p


MANY_ROUNDS = [
    # group, ranks in the pool, hin, T, adapters, dtype: each makes >= 16 rounds of shrink workgroups by the host's
    # count (slices of hin x min(T/group + adapters + 1, T rounded up to 8) records >= 16 x 768)
    (4, [8, 16, 32], 8192, 2048, 1200, FP16),
    (2, [8, 16, 32], 8192, 2048, 1200, FP16),
    (1, [16, 64], 8192, 2048, 600, BF16),
    (8, [8, 16], 16384, 4096, 1200, BF16),
    (8, [8, 16, 32], 8192, 2048, 1200, FP16),
]


@pytest.mark.parametrize("group,rank_set,hin,T,N,dtype", MANY_ROUNDS, ids=[f"g{c[0]}-r{max(c[1])}-{c[2]}" for c in MANY_ROUNDS])
def test_bgmv_many_round_launch_walks_several_records(group, rank_set, hin, T, N, dtype):
    """A launch of many rounds of workgroups (thousands of possible (record, slice) pairs) covers fewer records
    than the batch has in use, so every workgroup walks several records.  Mixed ranks in one pool (in a rank-32
    launch the rank-32 items take two shrink slices per workgroup), adapters with 64, 17 and 16 tokens next to
    hundreds with one to three, tokens without an adapter; accumulate and delta against the oracle, for each launch
    width (rank 16 / 32 / 64), token group and both dtypes."""
    rng = np.random.default_rng(4242 + group)
    hout = 1024
    ranks = rng.choice(rank_set, N)
    pp = PagedPool(rng, ranks, hin, hout, page_rows=8, dtype=dtype)
    ids = rng.permutation(N)
    rest = T - 148 - (N - 3)                                      # tokens left after one per remaining adapter
    tok = np.concatenate([np.repeat(ids[0], 64), np.repeat(ids[1], 17), np.repeat(ids[2], 16), np.full(51, -1),
                          ids[3:], rng.choice(ids[3:], rest)]).astype(np.int32)
    assert len(tok) == T
    tok = rng.permutation(tok)
    x = bits_of(rng.standard_normal((T, hin)).astype(np.float32), dtype)
    y0 = bits_of(rng.standard_normal((T, hout)).astype(np.float32), dtype)
    say(f"bgmv many-round launch, T={T}, {N} adapters of rank {rank_set}, hin={hin}, group={group}")
    got = _run(pp, x, tok, y0, group, accumulate=True, fused=False)
    assert_close_bits(got, oracle_apply(pp, x, tok, y0), dtype, "accumulate")
    got = _run(pp, x, tok, None, group, accumulate=False, fused=False)
    want = oracle_apply(pp, x, tok, None)
    assert_close_bits(got, want, dtype, "delta")
    assert not np.any(f32_of(got, dtype)[tok < 0]), "rows of tokens without an adapter must be zeros in y = delta mode"
