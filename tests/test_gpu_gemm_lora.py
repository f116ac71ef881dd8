"""GPU parity: base projection + LoRA in one pass (MFMA GEMM with the expand riding along) through the C ABI,
against the fp32-accumulated oracle (rtol 1e-2 / atol 1e-3), bit-exact on integer-valued inputs, and against
the library GEMM followed by the SGMV kernels at full config-4 width."""
import zlib

import numpy as np
import pytest
import torch

from gpu_common import ATOL, RTOL, assert_close_bits, say, tdtype, upload_pool
from helpers import BF16, FP16, PagedPool, bits_of, bits_to_torch, f32_of, torch_to_bits
from mlora import AdapterPool, gemm_lora, plan_prefill, sgmv_multi
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def _oracle(pp, x, w, tok, **kw):
    return orc.gemm_lora_paged(x, w, pp.a_rows, pp.b_rows, tok, pp.page_tbl, pp.page_tbl, pp.ranks, pp.scaling,
                               pp.page_rows, pp.dtype, **kw)


def _layout(lens, gaps, adapters):
    """Segments laid out one after another with `gaps[i]` adapter-less tokens before segment i."""
    start, pos = [], 0
    for l, g in zip(lens, gaps):
        pos += g
        start.append(pos)
        pos += l
    return np.asarray(start, np.int32), np.asarray(lens, np.int32), np.asarray(adapters, np.int32), pos


def _tok_of(start, lens, adapters, T):
    tok = np.full(T, -1, np.int32)
    for s, l, a in zip(start, lens, adapters):
        tok[s:s + l] = a
    return tok


def _run(pp, x_bits, w_bits, seg, T, aligned=False):
    pool = upload_pool(pp)
    x = bits_to_torch(x_bits, pp.dtype, "cuda")
    w = bits_to_torch(w_bits, pp.dtype, "cuda")
    y = torch.full((T, pp.hout), float("nan"), dtype=tdtype(pp.dtype), device="cuda")
    ss, sl, sa = (torch.from_numpy(a).cuda() for a in seg)
    plan = plan_prefill(ss, sl, sa, T, pool, aligned=aligned)
    gemm_lora([y], [x], [w], pool, 0, ["p"], plan)
    torch.cuda.synchronize()
    return torch_to_bits(y)


CASES = [
    # name, segment lengths, gaps before them, tail tokens, pool ranks, hin, hout, dtype
    ("q slice 1024x1024 fp16 r16", [70, 128, 1, 57], [0, 0, 0, 0], 0, [16] * 4, 1024, 1024, FP16),
    ("bf16 r64, K tail 1032x520, gaps", [37, 44, 51, 64, 100], [3, 0, 5, 0, 1], 7, [64, 24, 8], 1032, 520, BF16),
    ("rank 32 pool, ragged N 512x776", [64, 64, 64, 9], [0, 0, 0, 0], 0, [32, 17, 32], 512, 776, FP16),
    ("one K step and a tail 72x72", [5], [0], 0, [8], 72, 72, BF16),
    ("tail only 40x264", [30, 3], [2, 0], 1, [16, 4], 40, 264, FP16),
    ("three row tiles 640x256", [300, 250, 130], [0, 20, 0], 0, [16, 16], 640, 256, FP16),
]


@pytest.mark.parametrize("name,lens,gaps,tail,ranks,hin,hout,dtype", CASES, ids=[c[0] for c in CASES])
def test_gemm_lora_vs_oracle(name, lens, gaps, tail, ranks, hin, hout, dtype):
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    pp = PagedPool(rng, ranks, hin, hout, page_rows=8, dtype=dtype)
    adapters = rng.integers(0, len(ranks), len(lens))
    if len(lens) > 2:
        adapters[1] = -1                                   # a segment without adapter: base product only
    ss, sl, sa, T = _layout(lens, gaps, adapters)
    T += tail
    tok = _tok_of(ss, sl, sa, T)
    x = bits_of(rng.standard_normal((T, hin)).astype(np.float32), dtype)
    w = bits_of((rng.standard_normal((hin, hout)) / np.sqrt(hin)).astype(np.float32), dtype)
    say(f"gemm_lora {name}")
    got = _run(pp, x, w, (ss, sl, sa), T)
    assert_close_bits(got, _oracle(pp, x, w, tok), dtype, name)
    say(f"gemm_lora {name}, tiles cut at multiples of 64")
    assert_close_bits(_run(pp, x, w, (ss, sl, sa), T, aligned=True), _oracle(pp, x, w, tok), dtype, name + " aligned")
    # much closer than the tolerance: within one 16-bit ulp of the fp64 result (+ fp32 accumulation noise)
    want64 = f32_of(_oracle(pp, x, w, tok, acc64=True), dtype).astype(np.float64)
    err = np.abs(f32_of(got, dtype) - want64)
    mant = 10 if dtype == FP16 else 7
    assert np.all(err <= 2.0 ** -mant * np.abs(want64) + 2e-5), "not within one ulp of the exact result"


def test_gemm_lora_integer_inputs_bit_exact():
    rng = np.random.default_rng(81)
    ranks = [8, 16, 3, 64, 5]
    pp = PagedPool(rng, ranks, hin=512, hout=384, page_rows=8, dtype=FP16, integer=True)
    pp.scaling[:] = [1, 2, 0.5, -1, 4]
    lens, gaps = [33, 64, 65, 1, 130], [0, 2, 0, 0, 4]
    ss, sl, sa, T = _layout(lens, gaps, [4, 0, 1, 3, 2])
    tok = _tok_of(ss, sl, sa, T)
    xi = (rng.integers(-2, 3, (T, 512)) * (rng.random((T, 512)) < 0.05)).astype(np.float32)
    wi = (rng.integers(-1, 2, (512, 384)) * (rng.random((512, 384)) < 0.5)).astype(np.float32)
    x, w = bits_of(xi, FP16), bits_of(wi, FP16)
    want = _oracle(pp, x, w, tok)
    assert np.abs(f32_of(want, FP16)).max() < 2048
    say("gemm_lora integer-valued inputs")
    assert np.array_equal(_run(pp, x, w, (ss, sl, sa), T), want)
    assert np.array_equal(_run(pp, x, w, (ss, sl, sa), T, aligned=True), want)


@pytest.mark.parametrize("dtype", [FP16, BF16])
def test_gemm_base_only_matches_library_product(dtype):
    """No plan: the base products alone, against torch.mm in fp32 on the same 16-bit inputs."""
    torch.manual_seed(5)
    td = tdtype(dtype)
    T, hin, hout = 333, 1096, 840
    x = torch.randn(T, hin, device="cuda").to(td)
    w = (torch.randn(hin, hout, device="cuda") / hin ** 0.5).to(td)
    y = torch.full((T, hout), float("nan"), dtype=td, device="cuda")
    say(f"gemm base only {td}")
    gemm_lora([y], [x], [w], None, 0, ["p"], None)
    want = (x.float() @ w.float())
    err = (y.float() - want).abs()
    assert bool((err <= ATOL + RTOL * want.abs()).all())
    assert bool((err <= 2.0 ** (-10 if dtype == FP16 else -7) * want.abs() + 2e-5).all())


def test_gemm_lora_three_projections_one_launch():
    """q, k (same x) and a wider projection with its own x in one call, each against the oracle."""
    rng = np.random.default_rng(83)
    dims = {"q": (512, 512), "k": (512, 256), "g": (768, 1376)}
    ranks = [16, 8, 32]
    pps = {p: PagedPool(np.random.default_rng(90), ranks, hin, hout, page_rows=8, dtype=FP16) for p, (hin, hout) in dims.items()}
    first = pps["q"]
    pool = AdapterPool(1, dims, first.n, first.n_pages, page_rows=8, max_rank=32, dtype=torch.float16, device="cuda")
    pool.h_page_tbl[:] = first.page_tbl
    pool.h_rank[:] = first.ranks
    pool.h_scaling[:] = first.scaling
    pool._dirty = True
    pool.sync()
    for p, pp in pps.items():
        assert np.array_equal(pp.page_tbl, first.page_tbl)
        pool.a_rows[p][0].copy_(bits_to_torch(pp.a_rows, FP16))
        pool.b_rows[p][0].copy_(bits_to_torch(pp.b_rows, FP16))
    ss, sl, sa, T = _layout([100, 64, 200], [0, 3, 0], [2, 0, 1])
    tok = _tok_of(ss, sl, sa, T)
    xb = {512: bits_of(rng.standard_normal((T, 512)).astype(np.float32), FP16),
          768: bits_of(rng.standard_normal((T, 768)).astype(np.float32), FP16)}
    xt = {k: bits_to_torch(v, FP16, "cuda") for k, v in xb.items()}
    wb = {p: bits_of((rng.standard_normal(d) / np.sqrt(d[0])).astype(np.float32), FP16) for p, d in dims.items()}
    ws = [bits_to_torch(wb[p], FP16, "cuda") for p in dims]
    ys = [torch.full((T, d[1]), float("nan"), dtype=torch.float16, device="cuda") for d in dims.values()]
    plan = plan_prefill(*(torch.from_numpy(a).cuda() for a in (ss, sl, sa)), T, pool, n_proj=3)
    say("gemm_lora three projections")
    gemm_lora(ys, [xt[d[0]] for d in dims.values()], ws, pool, 0, list(dims), plan)
    torch.cuda.synchronize()
    for i, (p, d) in enumerate(dims.items()):
        assert_close_bits(torch_to_bits(ys[i]), _oracle(pps[p], xb[d[0]], wb[p], tok), FP16, p)


def test_gemm_lora_config4_width_against_library_products():
    """Full config-4 attention width (5120 x 5120, rank 64, bf16, 2048 tokens): the one-pass result against
    fp32 library products of the same 16-bit operands, within the tolerance; and the SGMV kernels' delta added
    to the base-only result reproduces it to the roundings involved."""
    torch.manual_seed(7)
    T, H, r, n_seg = 2048, 5120, 64, 8
    pool = AdapterPool(1, {"q": (H, H)}, n_seg, n_seg * 8 + 2, page_rows=8, max_rank=64, dtype=torch.bfloat16, device="cuda")
    AB = []
    for a in range(n_seg):
        pool.allocate(a, r, 0.5)
        AB.append(((torch.randn(H, r) * 0.02).bfloat16(), (torch.randn(r, H) * 0.02).bfloat16()))
        pool.load(a, 0, "q", *AB[-1])
    x = torch.randn(T, H, device="cuda").bfloat16()
    w = (torch.randn(H, H, device="cuda") / H ** 0.5).bfloat16()
    L = T // n_seg
    ss = torch.arange(0, T, L, dtype=torch.int32, device="cuda")
    sl = torch.full((n_seg,), L, dtype=torch.int32, device="cuda")
    sa = torch.arange(n_seg, dtype=torch.int32, device="cuda")
    plan = plan_prefill(ss, sl, sa, T, pool)
    y = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device="cuda")
    say("gemm_lora config-4 width, one pass")
    gemm_lora([y], [x], [w], pool, 0, ["q"], plan)
    ref = torch.mm(x.float(), w.float())
    for a in range(n_seg):
        A, B = (m.cuda().float() for m in AB[a])
        ref[a * L:(a + 1) * L] += 0.5 * ((x[a * L:(a + 1) * L].float() @ A) @ B)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y.float()).all())
    err = (y.float() - ref).abs()
    assert bool((err <= ATOL + RTOL * ref.abs()).all()), float(err.max())
    assert bool((err <= 2.0 ** -8 * ref.abs() + 1e-4).all()), "not within one bf16 ulp of the fp32 reference"
    say("base only + sgmv delta")
    yb = torch.empty_like(y)
    gemm_lora([yb], [x], [w], None, 0, ["q"], None)
    delta = torch.empty_like(y)
    sgmv_multi([delta], [x], pool, 0, ["q"], plan, accumulate=False)
    torch.cuda.synchronize()
    assert float(delta.float().abs().max()) > 0.05                      # the delta is not negligible here
    # three bf16 roundings (y, base, delta) apart at most
    assert bool(((y.float() - yb.float() - delta.float()).abs() <= 2.0 ** -7 * (ref.abs() + delta.float().abs()) + 1e-4).all())


@pytest.mark.parametrize("aligned", [False, True])
def test_plan_tile_list_matches_oracle(aligned):
    """The tile list the plan kernel writes (first words of the workspace: segment, first token and token count
    per tile, then the count) is the oracle's, bit for bit, in both cutting modes; and SGMV gives the same
    result with either plan."""
    rng = np.random.default_rng(91)
    lens = rng.integers(0, 300, 37).astype(np.int32)
    gaps = (rng.integers(0, 2, 37) * rng.integers(0, 50, 37)).astype(np.int32)
    ss, sl, sa, T = _layout(lens, gaps, rng.integers(-1, 3, 37))
    T += 5
    pp = PagedPool(rng, [16, 8, 4], 64, 64, page_rows=8, dtype=FP16)
    pool = upload_pool(pp)
    say(f"plan tile list aligned={aligned}")
    plan = plan_prefill(*(torch.from_numpy(a).cuda() for a in (ss, sl, sa)), T, pool, aligned=aligned)
    torch.cuda.synchronize()
    want_s, want_t0, want_n = orc.sgmv_plan(ss, sl, 64, aligned=aligned)
    max_tiles = T // 64 + 2 * len(lens) + 1
    words = plan.workspace[:(3 * max_tiles + 1) * 4].cpu().numpy().view(np.int32)
    n = int(words[3 * max_tiles])
    assert n == len(want_s)
    assert np.array_equal(words[:n], want_s)
    assert np.array_equal(words[max_tiles:max_tiles + n], want_t0)
    assert np.array_equal(words[2 * max_tiles:2 * max_tiles + n], want_n)
