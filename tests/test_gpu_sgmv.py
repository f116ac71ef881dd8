"""GPU parity: SGMV prefill kernels (MFMA) through the C ABI against the fp32-accumulated oracle, and
against the decode kernel at full config-4 size."""
import numpy as np
import pytest
import torch

from gpu_common import ATOL, RTOL, assert_close_bits, oracle_apply, say, tdtype, upload_pool
from helpers import BF16, FP16, PagedPool, bits_of, bits_to_torch, f32_of, torch_to_bits
from mlora import bgmv, plan_prefill, sgmv

pytestmark = pytest.mark.gpu


def _segments(lens, adapters):
    lens = np.asarray(lens, np.int32)
    start = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    return start, lens, np.asarray(adapters, np.int32)


def _tok_of(start, lens, adapters, T):
    tok = np.full(T, -1, np.int32)
    for s, l, a in zip(start, lens, adapters):
        tok[s:s + l] = a
    return tok


def _run(pp, x_bits, seg, y0_bits, accumulate=True):
    pool = upload_pool(pp)
    T = x_bits.shape[0]
    x = bits_to_torch(x_bits, pp.dtype, "cuda")
    y = bits_to_torch(y0_bits, pp.dtype, "cuda") if y0_bits is not None else \
        torch.full((T, pp.hout), float("nan"), dtype=tdtype(pp.dtype), device="cuda")
    ss, sl, sa = (torch.from_numpy(a).cuda() for a in seg)
    sgmv(y, x, pool, 0, "p", ss, sl, sa, accumulate=accumulate)
    torch.cuda.synchronize()
    return torch_to_bits(y)


CASES = [
    # name, segment lengths, ranks of the pool, hin, hout, dtype
    ("C4 slice q 5120x5120 bf16 r64", [70, 128, 1, 300, 64, 65], [64] * 8, 5120, 5120, BF16),
    ("C4 slice gate 5120x13824 bf16 r64", [130, 33], [64] * 4, 5120, 13824, BF16),
    ("C4 slice down 13824x5120 bf16 r64", [90, 17, 64], [64] * 4, 13824, 5120, BF16),
    ("fp16 hetero ranks 4096x4096", [40, 100, 7, 64, 129], [8, 16, 32, 64, 24], 4096, 4096, FP16),
    ("rank 16 pool 1024x2048", [63, 64, 65, 1], [16, 8, 16, 3], 1024, 2048, FP16),
    ("odd widths 200x72 bf16", [5, 70], [32, 5], 200, 72, BF16),
    ("tile boundaries 127/128/129 r32 2048x1024", [127, 128, 129, 63, 64, 65], [32, 32, 16, 32], 2048, 1024, FP16),
]


@pytest.mark.parametrize("name,lens,ranks,hin,hout,dtype", CASES, ids=[c[0] for c in CASES])
def test_sgmv_vs_oracle(name, lens, ranks, hin, hout, dtype):
    import zlib
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    pp = PagedPool(rng, ranks, hin, hout, page_rows=8, dtype=dtype)
    adapters = rng.integers(0, len(ranks), len(lens))
    seg = _segments(lens, adapters)
    T = int(np.sum(lens))
    tok = _tok_of(*seg, T)
    x = bits_of(rng.standard_normal((T, hin)).astype(np.float32), dtype)
    y0 = bits_of(rng.standard_normal((T, hout)).astype(np.float32), dtype)
    say(f"sgmv {name} accumulate")
    got = _run(pp, x, seg, y0)
    assert_close_bits(got, oracle_apply(pp, x, tok, y0), dtype, name)
    say(f"sgmv {name} delta")
    got_d = _run(pp, x, seg, None, accumulate=False)
    want_d = oracle_apply(pp, x, tok, None)
    assert_close_bits(got_d, want_d, dtype, name + " delta")
    # the hi+lo split keeps the intermediate at fp32 accuracy: the delta is much closer to the
    # fp64-accumulated oracle than a 16-bit intermediate would allow
    want64 = f32_of(oracle_apply(pp, x, tok, None, acc64=True), dtype).astype(np.float64)
    err = np.abs(f32_of(got_d, dtype) - want64)
    mant = 10 if dtype == FP16 else 7
    assert np.all(err <= 2.0 ** -mant * np.abs(want64) + 1e-5), "delta is not within one ulp of the exact result"


def test_sgmv_integer_inputs_bit_exact():
    rng = np.random.default_rng(71)
    ranks = [8, 16, 3, 64, 5]
    pp = PagedPool(rng, ranks, hin=512, hout=384, page_rows=8, dtype=FP16, integer=True)
    pp.scaling[:] = [1, 2, 0.5, -1, 4]
    lens = [64, 3, 100, 65, 1]
    seg = _segments(lens, [3, 0, 1, 2, 4])
    T = sum(lens)
    tok = _tok_of(*seg, T)
    xi = (rng.integers(-2, 3, (T, 512)) * (rng.random((T, 512)) < 0.05)).astype(np.float32)
    y0 = bits_of(rng.integers(-8, 9, (T, 384)).astype(np.float32), FP16)
    x = bits_of(xi, FP16)
    want = oracle_apply(pp, x, tok, y0)
    assert np.abs(f32_of(want, FP16)).max() < 2048
    say("sgmv integer-valued inputs")
    assert np.array_equal(_run(pp, x, seg, y0), want)


def test_sgmv_segments_without_adapter_and_gaps():
    rng = np.random.default_rng(72)
    pp = PagedPool(rng, [16, 32], 256, 256, page_rows=8, dtype=FP16)
    # tokens 0..9 uncovered, then a segment with no adapter, an empty one, and two real ones
    ss = np.array([10, 40, 40, 104], np.int32)
    sl = np.array([30, 0, 64, 20], np.int32)
    sa = np.array([-1, 1, 0, 1], np.int32)
    T = 130
    tok = _tok_of(ss, sl, sa, T)
    x = bits_of(rng.standard_normal((T, 256)).astype(np.float32), FP16)
    y0 = bits_of(rng.standard_normal((T, 256)).astype(np.float32), FP16)
    say("sgmv gaps / adapter-less segment, accumulate")
    got = _run(pp, x, (ss, sl, sa), y0)
    assert np.array_equal(got[tok < 0], y0[tok < 0])
    assert_close_bits(got, oracle_apply(pp, x, tok, y0), FP16)
    say("sgmv gaps / adapter-less segment, delta")
    got_d = _run(pp, x, (ss, sl, sa), None, accumulate=False)
    assert np.all(got_d[10:40] == 0)                       # adapter-less segment is defined as zeros
    assert np.all(got_d[tok < 0] == 0)                     # ... and so are tokens 0..9 and 124..129, which no segment covers
    assert_close_bits(got_d, oracle_apply(pp, x, tok, None), FP16)


def test_sgmv_delta_defines_rows_outside_every_segment():
    """y = delta mode over NaN-filled memory: rows between, before and after the segments (given out of
    order) come back as zeros from the one-projection, the planned and the multi-projection calls."""
    from mlora import plan_prefill, sgmv, sgmv_multi
    rng = np.random.default_rng(75)
    hin, hout = 256, 392
    pp = PagedPool(rng, [8, 64, 24], hin, hout, page_rows=8, dtype=BF16)
    ss = np.array([200, 5, 70], np.int32)                  # gaps: 0..4, 69, 135..199, 263..299
    sl = np.array([63, 64, 65], np.int32)
    sa = np.array([2, 0, 1], np.int32)
    T = 300
    tok = _tok_of(ss, sl, sa, T)
    x = bits_of(rng.standard_normal((T, hin)).astype(np.float32), BF16)
    want = oracle_apply(pp, x, tok, None)
    assert np.all(want[tok < 0] == 0) and (tok < 0).sum() == 108
    say("sgmv delta with gaps: self-planning call")
    got = _run(pp, x, (ss, sl, sa), None, accumulate=False)
    assert np.all(got[tok < 0] == 0)
    assert_close_bits(got, want, BF16)
    pool = upload_pool(pp)
    seg = tuple(torch.from_numpy(a).cuda() for a in (ss, sl, sa))
    xt = bits_to_torch(x, BF16, "cuda")
    plan = plan_prefill(*seg, T, pool, n_proj=2)
    nan = lambda: torch.full((T, hout), float("nan"), dtype=torch.bfloat16, device="cuda")
    say("sgmv delta with gaps: planned and multi-projection calls")
    y1, y2, y3 = nan(), nan(), nan()
    sgmv(y1, xt, pool, 0, "p", accumulate=False, plan=plan)
    sgmv_multi([y2, y3], [xt, xt], pool, 0, ["p", "p"], plan, accumulate=False)
    torch.cuda.synchronize()
    for y in (y1, y2, y3):
        bits = torch_to_bits(y)
        assert np.all(bits[tok < 0] == 0)
        assert_close_bits(bits, want, BF16)


def test_sgmv_plan_once_apply_many():
    """One plan serves several projections and layers, and matches the self-planning call bit for bit."""
    rng = np.random.default_rng(73)
    ranks = [64, 16, 32, 8]
    hin, hout = 512, 768
    pp = PagedPool(rng, ranks, hin, hout, page_rows=8, dtype=BF16)
    from mlora import AdapterPool
    pool = upload_pool(pp, projections={"p": (hin, hout), "o": (hout, hin)}, n_layers=2)
    for l in range(2):
        pool.a_rows["o"][l].normal_(0, 0.02)
        pool.b_rows["o"][l].normal_(0, 0.02)
    pool.a_rows["p"][1].normal_(0, 0.02)
    pool.b_rows["p"][1].normal_(0, 0.02)
    lens = [70, 3, 128, 65]
    ss, sl, sa = (torch.from_numpy(a).cuda() for a in _segments(lens, [2, 0, 3, 1]))
    T = sum(lens)
    say("sgmv: one plan, two layers x two projections")
    plan = plan_prefill(ss, sl, sa, T, pool)
    for l in range(2):
        for proj, (hi, ho) in (("p", (hin, hout)), ("o", (hout, hin))):
            x = torch.randn(T, hi, device="cuda").bfloat16()
            y0 = torch.randn(T, ho, device="cuda").bfloat16()
            y_plan, y_self = y0.clone(), y0.clone()
            sgmv(y_plan, x, pool, l, proj, plan=plan)
            sgmv(y_self, x, pool, l, proj, ss, sl, sa)
            torch.cuda.synchronize()
            assert torch.equal(y_plan, y_self)
            assert not torch.equal(y_plan, y0)


def test_sgmv_equals_bgmv_at_config4_size():
    """Config 4 at full size (16 requests, lengths U[128,1024], 32 rank-64 adapters, hidden 5120, bf16):
    the prefill kernels and the decode kernel must agree within tolerance on every token."""
    rng = np.random.default_rng(1004)
    lens = rng.integers(128, 1025, 16)
    adapters = rng.integers(0, 32, 16)
    seg = _segments(lens, adapters)
    T = int(lens.sum())
    pp = PagedPool(rng, [64] * 32, 5120, 5120, page_rows=8, dtype=BF16)
    pool = upload_pool(pp)
    x = (torch.randn(T, 5120, device="cuda")).to(torch.bfloat16)
    y0 = (torch.randn(T, 5120, device="cuda")).to(torch.bfloat16)
    tok = torch.from_numpy(_tok_of(*seg, T)).cuda()
    ys, yb = y0.clone(), y0.clone()
    say(f"sgmv vs bgmv at config-4 size T={T}")
    sgmv(ys, x, pool, 0, "p", *(torch.from_numpy(a).cuda() for a in seg))
    bgmv([yb], [x], pool, 0, ["p"], tok)
    torch.cuda.synchronize()
    assert torch.allclose(ys.float(), yb.float(), rtol=RTOL, atol=ATOL)
    # linearity of the delta in x at full size
    d1, d2 = torch.zeros_like(y0), torch.zeros_like(y0)
    sgmv(d1, x, pool, 0, "p", *(torch.from_numpy(a).cuda() for a in seg), accumulate=False)
    sgmv(d2, (2 * x).contiguous(), pool, 0, "p", *(torch.from_numpy(a).cuda() for a in seg), accumulate=False)
    torch.cuda.synchronize()
    assert torch.equal(d2, 2 * d1)


def test_sgmv_multi_projection_call():
    """q, k, v (one x) and o (own x, other widths) in one call of three launches: every projection against the
    oracle, bit for bit on integer-valued inputs, and no effect on rows outside the segments."""
    from mlora import sgmv_multi
    rng = np.random.default_rng(74)
    ranks = [64, 16, 32, 8, 24]
    shapes = {"q": (512, 512), "k": (512, 256), "v": (512, 256), "o": (768, 512)}
    ss = np.array([5, 75, 78, 78, 206], np.int32)
    sl = np.array([70, 3, 0, 128, 65], np.int32)
    sa = np.array([2, 0, 1, 3, -1], np.int32)
    T = 280
    tok = _tok_of(ss, sl, sa, T)
    for integer in (False, True):
        pps = {p: PagedPool(np.random.default_rng(80), ranks, hin, hout, page_rows=8, dtype=FP16, integer=integer)
               for p, (hin, hout) in shapes.items()}
        for i, p in enumerate(shapes):                # same page table, different weights per projection
            r2 = np.random.default_rng(90 + i)
            if integer:
                pps[p].a_rows = bits_of(r2.integers(-2, 3, pps[p].a_rows.shape).astype(np.float32), FP16)
                pps[p].b_rows = bits_of(r2.integers(-2, 3, pps[p].b_rows.shape).astype(np.float32), FP16)
                pps[p].scaling[:] = [1, 2, 0.5, -1, 4]
            else:
                pps[p].a_rows = bits_of((r2.standard_normal(pps[p].a_rows.shape) * 0.02).astype(np.float32), FP16)
                pps[p].b_rows = bits_of((r2.standard_normal(pps[p].b_rows.shape) * 0.02).astype(np.float32), FP16)
        pool = upload_pool(pps["q"], projections=shapes)
        pool.h_scaling[:] = pps["q"].scaling
        pool._dirty = True
        for p in shapes:
            pool.a_rows[p][0].copy_(bits_to_torch(pps[p].a_rows, FP16))
            pool.b_rows[p][0].copy_(bits_to_torch(pps[p].b_rows, FP16))
        if integer:
            mk = lambda h: bits_of((rng.integers(-2, 3, (T, h)) * (rng.random((T, h)) < 0.04)).astype(np.float32), FP16)
            y0 = {p: bits_of(rng.integers(-8, 9, (T, shapes[p][1])).astype(np.float32), FP16) for p in shapes}
        else:
            mk = lambda h: bits_of(rng.standard_normal((T, h)).astype(np.float32), FP16)
            y0 = {p: bits_of(rng.standard_normal((T, shapes[p][1])).astype(np.float32), FP16) for p in shapes}
        x_qkv, x_o = mk(512), mk(768)
        xt_qkv, xt_o = bits_to_torch(x_qkv, FP16, "cuda"), bits_to_torch(x_o, FP16, "cuda")
        ys = {p: bits_to_torch(y0[p], FP16, "cuda") for p in shapes}
        d = [torch.from_numpy(a).cuda() for a in (ss, sl, sa)]
        plan = plan_prefill(d[0], d[1], d[2], T, pool, n_proj=4)
        say(f"sgmv_multi q,k,v,o integer={integer}")
        sgmv_multi([ys[p] for p in "qkvo"], [xt_qkv, xt_qkv, xt_qkv, xt_o], pool, 0, list("qkvo"), plan)
        torch.cuda.synchronize()
        for p in "qkvo":
            pps[p].scaling[:] = pps["q"].scaling
            want = oracle_apply(pps[p], x_o if p == "o" else x_qkv, tok, y0[p])
            got = torch_to_bits(ys[p])
            assert np.array_equal(got[tok < 0], y0[p][tok < 0])
            if integer:
                assert np.abs(f32_of(want, FP16)).max() < 2048
                assert np.array_equal(got, want), p
            else:
                assert_close_bits(got, want, FP16, f"projection {p}")
        # the same plan still serves single-projection calls
        y1 = bits_to_torch(y0["k"], FP16, "cuda")
        sgmv(y1, xt_qkv, pool, 0, "k", plan=plan)
        torch.cuda.synchronize()
        if integer:
            assert torch.equal(y1, ys["k"])
        else:
            assert torch.allclose(y1.float(), ys["k"].float(), rtol=RTOL, atol=ATOL)
