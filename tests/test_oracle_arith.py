"""Pins the oracle's arithmetic: exact rational brute force on tiny cases, integer-valued inputs
(where every fp32 operation is exact, so any correct implementation is bit-identical whatever its
summation order), library matmuls, closed-form special cases and invariants."""
from fractions import Fraction

import numpy as np
import pytest
import torch

from helpers import BF16, FP16, PagedPool, bits_of, exact_round16, f32_of, ulp16
from oracle import oracle as orc


def _apply(pool, x_bits, tok, y0_bits=None, acc64=False):
    return orc.lora_apply_paged(x_bits, pool.a_rows, pool.b_rows, tok, pool.page_tbl, pool.page_tbl, pool.ranks,
                                pool.scaling, pool.page_rows, pool.dtype, y0=y0_bits, acc64=acc64)


@pytest.mark.parametrize("dtype", [FP16, BF16])
def test_exact_rational_brute_force(dtype):
    rng = np.random.default_rng(10 + dtype)
    pool = PagedPool(rng, [1, 3, 4, 2], hin=16, hout=24, page_rows=2, dtype=dtype, std=0.5)
    T = 4
    tok = np.array([2, 0, 3, 1], np.int32)
    x = bits_of(rng.standard_normal((T, 16)).astype(np.float32), dtype)
    y0 = bits_of(rng.standard_normal((T, 24)).astype(np.float32), dtype)
    got = _apply(pool, x, tok, y0, acc64=True)
    got32 = _apply(pool, x, tok, y0, acc64=False)
    xf, y0f = f32_of(x, dtype), f32_of(y0, dtype)
    n_equal = 0
    for t in range(T):
        a = int(tok[t])
        rows = pool.rows(a)
        A = f32_of(pool.a_rows[rows], dtype)     # [r, Hin]
        B = f32_of(pool.b_rows[rows], dtype)     # [r, Hout]
        s = Fraction(float(pool.scaling[a]))
        v = [sum(Fraction(float(xf[t, k])) * Fraction(float(A[j, k])) for k in range(16)) for j in range(len(rows))]
        for c in range(24):
            exact = Fraction(float(y0f[t, c])) + s * sum(v[j] * Fraction(float(B[j, c])) for j in range(len(rows)))
            want = exact_round16(exact, dtype)
            n_equal += int(got[t, c]) == want
            w = f32_of(np.array([want], np.uint16), dtype)[0]
            u = ulp16(np.array([w]), dtype)[0]
            assert abs(float(f32_of(got[t:t + 1, c], dtype)[0]) - w) <= u
            assert abs(float(f32_of(got32[t:t + 1, c], dtype)[0]) - w) <= u
    assert n_equal >= 0.98 * T * 24      # fp64 accumulation rounds like the exact value except at near-ties


@pytest.mark.parametrize("dtype", [FP16, BF16])
@pytest.mark.parametrize("page_rows", [1, 8])
def test_integer_inputs_bit_exact_vs_int_matmul(dtype, page_rows):
    rng = np.random.default_rng(20 + page_rows)
    ranks = [8, 16, 3, 1, 5]
    pool = PagedPool(rng, ranks, hin=64, hout=40, page_rows=page_rows, dtype=dtype, integer=True)
    pool.scaling[:] = [1, 2, 0.5, -1, 4]
    T = 23
    tok = rng.integers(-1, len(ranks), T).astype(np.int32)
    xi = rng.integers(-2, 3, (T, 64))
    y0i = rng.integers(-8, 9, (T, 40))
    y = _apply(pool, bits_of(xi.astype(np.float32), dtype), tok, bits_of(y0i.astype(np.float32), dtype))
    want = y0i.astype(np.float64)
    for t in range(T):
        if tok[t] >= 0:
            a = int(tok[t])
            want[t] += pool.scaling[a] * (xi[t].astype(np.float64) @ pool.A(a) @ pool.B(a))
    assert np.abs(want).max() < (2048 if dtype == FP16 else 256)   # exactly representable
    assert np.array_equal(f32_of(y, dtype).astype(np.float64), want)
    # y = delta form
    yd = _apply(pool, bits_of(xi.astype(np.float32), dtype), tok, None)
    assert np.array_equal(f32_of(yd, dtype).astype(np.float64), want - y0i)


def test_scale_zero_and_no_adapter_keep_y0():
    rng = np.random.default_rng(30)
    pool = PagedPool(rng, [16, 8], hin=32, hout=32)
    pool.scaling[:] = 0.0
    x = bits_of(rng.standard_normal((6, 32)).astype(np.float32), FP16)
    y0 = bits_of(rng.standard_normal((6, 32)).astype(np.float32), FP16)
    y = _apply(pool, x, np.array([0, 1, -1, 0, -1, 1], np.int32), y0)
    assert np.array_equal(y, y0)


def test_one_hot_picks_a_row_times_b():
    rng = np.random.default_rng(31)
    pool = PagedPool(rng, [4, 16], hin=32, hout=48, std=0.3)
    k = 7
    x = np.zeros((1, 32), np.float32)
    x[0, k] = 1.0
    y = f32_of(_apply(pool, bits_of(x, FP16), np.array([1], np.int32), None, acc64=True), FP16)
    want = pool.scaling[1] * (pool.A(1)[k, :] @ pool.B(1))
    assert np.all(np.abs(y[0] - want) <= ulp16(want, FP16))


@pytest.mark.parametrize("dtype", [FP16, BF16])
def test_single_adapter_reduces_to_two_matmuls(dtype):
    rng = np.random.default_rng(32)
    pool = PagedPool(rng, [16], hin=256, hout=128, dtype=dtype)
    x = bits_of(rng.standard_normal((9, 256)).astype(np.float32), dtype)
    y0 = bits_of(rng.standard_normal((9, 128)).astype(np.float32), dtype)
    y = f32_of(_apply(pool, x, np.zeros(9, np.int32), y0), dtype).astype(np.float64)
    want = f32_of(y0, dtype) + pool.scaling[0] * (f32_of(x, dtype).astype(np.float64) @ pool.A(0) @ pool.B(0))
    assert np.all(np.abs(y - want) <= 1.01 * ulp16(want, dtype))


def test_invariants_pages_permutation_padding_linearity():
    rng = np.random.default_rng(33)
    ranks = [8, 32, 16, 64]
    T, hin, hout = 12, 64, 64
    p1 = PagedPool(np.random.default_rng(1), ranks, hin, hout, shuffle=True)
    tok = rng.integers(0, 4, T).astype(np.int32)
    x = bits_of(rng.standard_normal((T, hin)).astype(np.float32), FP16)
    y0 = bits_of(rng.standard_normal((T, hout)).astype(np.float32), FP16)
    y1 = _apply(p1, x, tok, y0)
    # same weights placed on other pages -> identical bits
    p2 = PagedPool(np.random.default_rng(2), ranks, hin, hout, shuffle=True, extra_pages=11)
    for i in range(4):
        p2.a_rows[p2.rows(i)] = p1.a_rows[p1.rows(i)]
        p2.b_rows[p2.rows(i)] = p1.b_rows[p1.rows(i)]
    assert np.array_equal(_apply(p2, x, tok, y0), y1)
    # permuting tokens permutes outputs
    perm = rng.permutation(T)
    assert np.array_equal(_apply(p1, x[perm], tok[perm], y0[perm]), y1[perm])
    # rank-8 adapter stored in a 64-row allocation with zero rows beyond 8 -> identical
    p3 = PagedPool(np.random.default_rng(3), [64, 32, 16, 64], hin, hout)
    for i in range(1, 4):
        p3.a_rows[p3.rows(i)] = p1.a_rows[p1.rows(i)]
        p3.b_rows[p3.rows(i)] = p1.b_rows[p1.rows(i)]
    r3 = p3.rows(0)
    p3.a_rows[r3] = 0
    p3.b_rows[r3] = 0
    p3.a_rows[r3[:8]] = p1.a_rows[p1.rows(0)]
    p3.b_rows[r3[:8]] = p1.b_rows[p1.rows(0)]
    p3.scaling[:] = p1.scaling
    assert np.array_equal(_apply(p3, x, tok, y0), y1)
    # the delta is linear in x: delta(2x) == 2 delta(x) exactly (power-of-two scaling)
    d1 = f32_of(_apply(p1, x, tok, None), FP16)
    x2 = bits_of(2 * f32_of(x, FP16), FP16)
    d2 = f32_of(_apply(p1, x2, tok, None), FP16)
    normal = np.abs(d1) >= 2.0 ** -13            # doubling is exact only outside the subnormal range
    assert normal.mean() > 0.9 and np.array_equal(d2[normal], 2 * d1[normal])


def test_reflayout_call_equals_paged_call():
    """add_lora_bgmv on [N,L,r,Hin]/[N,L,Hout,r] (lora_gpu.py:33-40,138) is the paged apply on the same weights."""
    rng = np.random.default_rng(34)
    N, L, r, hin, hout, T, layer = 5, 3, 16, 64, 48, 10, 1
    wa = bits_of((rng.standard_normal((N, L, r, hin)) * 0.1).astype(np.float32), FP16)
    wb = bits_of((rng.standard_normal((N, L, hout, r)) * 0.1).astype(np.float32), FP16)
    idx = rng.integers(0, N, T).astype(np.int64)
    x = bits_of(rng.standard_normal((T, hin)).astype(np.float32), FP16)
    y0 = bits_of(rng.standard_normal((T, hout)).astype(np.float32), FP16)
    y = y0.copy()
    orc.add_lora_bgmv_ref(y, x, wa, wb, idx, layer, 0.75)
    # equivalent paged pool: adapter i owns rows [i*r, (i+1)*r)
    a_rows = np.ascontiguousarray(wa[:, layer].reshape(N * r, hin))
    b_rows = np.ascontiguousarray(wb[:, layer].transpose(0, 2, 1).reshape(N * r, hout))
    tbl = (np.arange(N, dtype=np.int32) * (r // 8))[:, None] + np.arange(r // 8, dtype=np.int32)[None, :]
    yp = orc.lora_apply_paged(x, a_rows, b_rows, idx.astype(np.int32), tbl, tbl, np.full(N, r, np.int32),
                              np.full(N, 0.75, np.float32), 8, FP16, y0=y0)
    assert np.array_equal(y, yp)
    # and the expression itself through numpy in fp64
    want = f32_of(y0, FP16).astype(np.float64)
    for t in range(T):
        A = f32_of(wa[idx[t], layer], FP16).astype(np.float64)      # [r, Hin]
        B = f32_of(wb[idx[t], layer], FP16).astype(np.float64)      # [Hout, r]
        want[t] += 0.75 * (f32_of(x[t], FP16).astype(np.float64) @ A.T @ B.T)
    assert np.all(np.abs(f32_of(y, FP16) - want) <= 1.01 * ulp16(want, FP16))
    with pytest.raises(IndexError):
        orc.add_lora_bgmv_ref(y, x, wa, wb, np.full(T, N, np.int64), layer, 1.0)


def test_prefill_bmm_is_torch_bmm():
    """lora_gpu.py:127-128 evaluated by torch on the CPU in fp32 (same expression, library matmul)."""
    rng = np.random.default_rng(35)
    Bsz, Lpad, L, r, hin, hout, layer = 3, 7, 2, 8, 64, 32, 1
    A_T = (rng.standard_normal((Bsz, L, r, hin)) * 0.1).astype(np.float16)
    B_T = (rng.standard_normal((Bsz, L, hout, r)) * 0.1).astype(np.float16)
    x = rng.standard_normal((Bsz, Lpad, hin)).astype(np.float16)
    y = orc.prefill_bmm_ref(x.view(np.uint16), A_T.view(np.uint16), B_T.view(np.uint16), layer, FP16, round_mid=False)
    tx, tA, tB = (torch.from_numpy(a.astype(np.float32)) for a in (x, A_T, B_T))
    want = torch.bmm(torch.bmm(tx, tA[:Bsz, layer].transpose(-1, -2)), tB[:Bsz, layer].transpose(-1, -2)).numpy()
    got = f32_of(y, FP16)
    assert np.all(np.abs(got - want) <= 1.01 * ulp16(want, FP16) + 1e-7)
    # with the fp16 intermediate the reference's two half-precision bmm calls produce
    mid = torch.bmm(tx, tA[:Bsz, layer].transpose(-1, -2)).to(torch.float16).to(torch.float32)
    want2 = torch.bmm(mid, tB[:Bsz, layer].transpose(-1, -2)).numpy()
    got2 = f32_of(orc.prefill_bmm_ref(x.view(np.uint16), A_T.view(np.uint16), B_T.view(np.uint16), layer, FP16,
                                      round_mid=True), FP16)
    assert np.all(np.abs(got2 - want2) <= 1.01 * ulp16(want2, FP16) + 1e-7)


def test_cpu_worker_is_x_float_down_up_half():
    """lora_cpu/lora_shm_op/app.py:136-141: res = x.float() @ down @ up; out = res.half()."""
    rng = np.random.default_rng(36)
    hin, hout, r, n = 128, 96, 16, 5
    down = (rng.standard_normal((hin, r)) * 0.001).astype(np.float32)
    up = (rng.standard_normal((r, hout)) * 0.001).astype(np.float32)
    x = rng.standard_normal((n, hin)).astype(np.float16)
    got = orc.cpu_lora_worker(x.view(np.uint16), down, up).view(np.float16).astype(np.float64)
    want = (torch.from_numpy(x).float() @ torch.from_numpy(down) @ torch.from_numpy(up)).half().numpy().astype(np.float64)
    exact = x.astype(np.float64) @ down.astype(np.float64) @ up.astype(np.float64)
    assert np.all(np.abs(got - exact) <= 0.51 * ulp16(exact, FP16) + 1e-9)
    assert np.all(np.abs(got - want) <= ulp16(exact, FP16))
    # integer-valued inputs: bit-exact whatever the summation order
    xi = rng.integers(-2, 3, (n, hin)).astype(np.float16)
    di = rng.integers(-1, 2, (hin, r)).astype(np.float32)
    ui = rng.integers(-1, 2, (r, hout)).astype(np.float32)
    got = orc.cpu_lora_worker(xi.view(np.uint16), di, ui).view(np.float16).astype(np.float64)
    assert np.array_equal(got, xi.astype(np.float64) @ di @ ui)


@pytest.mark.parametrize("n_threads", [1, 3])
def test_cpu_batch_is_worker_per_chunk(n_threads):
    rng = np.random.default_rng(37)
    batch, tkn, cap, hin, hout, r, N = 3, 20, 8, 64, 32, 4, 5
    down = (rng.standard_normal((N, hin, r)) * 0.05).astype(np.float32)
    up = (rng.standard_normal((N, r, hout)) * 0.05).astype(np.float32)
    x = rng.standard_normal((batch * tkn, hin)).astype(np.float16).view(np.uint16)
    req_adapter = np.array([4, 0, 2], np.int32)
    got = orc.cpu_lora_batch(x, down, up, req_adapter, tkn, cap, n_threads)
    for b in range(batch):
        a = req_adapter[b]
        want = orc.cpu_lora_worker(x[b * tkn:(b + 1) * tkn], down[a], up[a])
        assert np.array_equal(got[b * tkn:(b + 1) * tkn], want)


def test_cpu_pool_equals_batch_over_many_wakeups():
    """The persistent worker pool gives the same bits as the spawn-per-call form, batch after batch."""
    rng = np.random.default_rng(38)
    hin, hout, r, N = 64, 48, 8, 6
    down = (rng.standard_normal((N, hin, r)) * 0.05).astype(np.float32)
    up = (rng.standard_normal((N, r, hout)) * 0.05).astype(np.float32)
    pool = orc.CpuLoraPool(3)
    try:
        for batch, tkn, cap in [(3, 20, 8), (1, 1, 8), (7, 5, 2), (4, 16, 16), (2, 9, 4)] * 3:
            x = rng.standard_normal((batch * tkn, hin)).astype(np.float16).view(np.uint16)
            req_adapter = rng.integers(0, N, batch).astype(np.int32)
            assert np.array_equal(pool.run(x, down, up, req_adapter, tkn, cap),
                                  orc.cpu_lora_batch(x, down, up, req_adapter, tkn, cap, 2))
    finally:
        pool.close()


# ---------------------------------------------------------------- base projection + LoRA (one pass)
def _gemm_lora(pool, x_bits, w_bits, tok, **kw):
    return orc.gemm_lora_paged(x_bits, w_bits, pool.a_rows, pool.b_rows, tok, pool.page_tbl, pool.page_tbl, pool.ranks,
                               pool.scaling, pool.page_rows, pool.dtype, **kw)


@pytest.mark.parametrize("dtype", [FP16, BF16])
def test_gemm_lora_integer_inputs_bit_exact(dtype):
    """Integer-valued operands: base product, delta and their sum are exact in fp32 and representable, so the
    single-rounding contract, the reference's three roundings and numpy's integer matmul must all agree."""
    rng = np.random.default_rng(70)
    ranks = [8, 3, 16, 1]
    pool = PagedPool(rng, ranks, hin=48, hout=40, page_rows=4, dtype=dtype, integer=True)
    pool.scaling[:] = [1, 2, 0.5, -1]
    T = 21
    tok = rng.integers(-1, len(ranks), T).astype(np.int32)
    xi = rng.integers(-2, 3, (T, 48)) * (rng.random((T, 48)) < 0.3)
    wi = rng.integers(-1, 2, (48, 40))
    want = (xi @ wi).astype(np.float64)
    for t in range(T):
        if tok[t] >= 0:
            a = int(tok[t])
            want[t] += pool.scaling[a] * (xi[t].astype(np.float64) @ pool.A(a) @ pool.B(a))
    assert np.abs(want).max() < (2048 if dtype == FP16 else 256)
    xb, wb = bits_of(xi.astype(np.float32), dtype), bits_of(wi.astype(np.float32), dtype)
    for kw in (dict(), dict(acc64=True), dict(ref_rounding=True), dict(acc64=True, ref_rounding=True)):
        assert np.array_equal(f32_of(_gemm_lora(pool, xb, wb, tok, **kw), dtype).astype(np.float64), want), kw


@pytest.mark.parametrize("dtype", [FP16, BF16])
def test_gemm_lora_is_library_matmul_plus_delta(dtype):
    rng = np.random.default_rng(71)
    pool = PagedPool(rng, [16, 8, 24], hin=256, hout=96, dtype=dtype)
    T = 17
    tok = rng.integers(-1, 3, T).astype(np.int32)
    x = bits_of(rng.standard_normal((T, 256)).astype(np.float32), dtype)
    w = bits_of((rng.standard_normal((256, 96)) * 0.05).astype(np.float32), dtype)
    xf, wf = f32_of(x, dtype).astype(np.float64), f32_of(w, dtype).astype(np.float64)
    want = xf @ wf
    for t in range(T):
        if tok[t] >= 0:
            a = int(tok[t])
            want[t] += pool.scaling[a] * (xf[t] @ pool.A(a) @ pool.B(a))
    got64 = f32_of(_gemm_lora(pool, x, w, tok, acc64=True), dtype).astype(np.float64)
    assert np.all(np.abs(got64 - want) <= 0.51 * ulp16(want, dtype))            # fp64 sums, one rounding
    got32 = f32_of(_gemm_lora(pool, x, w, tok), dtype).astype(np.float64)
    assert np.all(np.abs(got32 - want) <= 1.01 * ulp16(want, dtype) + 1e-5)     # fp32 sums over 256 terms
    # the reference's three roundings: half an ulp each of the base product, the delta and their sum
    got_ref = f32_of(_gemm_lora(pool, x, w, tok, ref_rounding=True, acc64=True), dtype).astype(np.float64)
    base, delta = xf @ wf, want - xf @ wf
    bound = 0.51 * (ulp16(base, dtype) + ulp16(delta, dtype) + ulp16(want, dtype)) + 0.51 * ulp16(got_ref, dtype)
    assert np.all(np.abs(got_ref - want) <= bound)
    assert np.any(got_ref != got64)                                              # and they do differ from one rounding
    # without adapters it is the plain product; the delta alone is what lora_apply_paged computes
    none = np.full(T, -1, np.int32)
    base = f32_of(_gemm_lora(pool, x, w, none, acc64=True), dtype).astype(np.float64)
    assert np.all(np.abs(base - xf @ wf) <= 0.51 * ulp16(xf @ wf, dtype))


def test_gemm_lora_zero_weight_equals_lora_apply():
    """W = 0 leaves the delta: bit-identical to the LoRA-only oracle with y = delta."""
    rng = np.random.default_rng(72)
    pool = PagedPool(rng, [16, 5], hin=128, hout=64, dtype=FP16)
    T = 11
    tok = rng.integers(-1, 2, T).astype(np.int32)
    x = bits_of(rng.standard_normal((T, 128)).astype(np.float32), FP16)
    w0 = np.zeros((128, 64), np.uint16)
    assert np.array_equal(_gemm_lora(pool, x, w0, tok), _apply(pool, x, tok, None))
