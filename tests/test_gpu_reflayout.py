"""GPU parity on the reference's own pool layout and call signatures (lightllm/models/lora_gpu.py)."""
import numpy as np
import pytest
import torch

from gpu_common import ATOL, RTOL, assert_close_bits, say
from helpers import BF16, FP16, bits_of, bits_to_torch, f32_of, torch_to_bits
from mlora import Lora_GPU, add_lora_bgmv, lora_prefill_ref
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("N,L,r,hin,hout,T,layer,scale,dtype", [
    (24, 4, 64, 4096, 4096, 17, 2, 1.0, FP16),       # the shipped shapes (rank 64, hidden 4096), fewer layers
    (8, 2, 16, 4096, 4096, 32, 0, 2.0, FP16),        # config 1
    (5, 3, 16, 512, 1536, 9, 1, 0.5, BF16),
    (4, 2, 12, 256, 264, 6, 1, 1.0, FP16),           # rank not a multiple of 8
    (3, 1, 2, 128, 128, 5, 0, 1.0, FP16),            # the CPU worker's default rank
])
def test_add_lora_bgmv_vs_oracle(N, L, r, hin, hout, T, layer, scale, dtype):
    rng = np.random.default_rng(N * 100 + r)
    wa = bits_of((rng.standard_normal((N, L, r, hin)) * 0.02).astype(np.float32), dtype)
    wb = bits_of((rng.standard_normal((N, L, hout, r)) * 0.02).astype(np.float32), dtype)
    idx = rng.integers(0, N, T).astype(np.int64)
    x = bits_of(rng.standard_normal((T, hin)).astype(np.float32), dtype)
    y0 = bits_of(rng.standard_normal((T, hout)).astype(np.float32), dtype)
    want = y0.copy()
    orc.add_lora_bgmv_ref(want, x, wa, wb, idx, layer, scale, dtype)
    y = bits_to_torch(y0, dtype, "cuda")
    say(f"add_lora_bgmv N={N} L={L} r={r} {hin}x{hout} T={T}")
    add_lora_bgmv(y, bits_to_torch(x, dtype, "cuda"), bits_to_torch(wa, dtype, "cuda"), bits_to_torch(wb, dtype, "cuda"),
                  torch.from_numpy(idx).cuda(), layer, scale)
    torch.cuda.synchronize()
    assert_close_bits(torch_to_bits(y), want, dtype)


@pytest.mark.parametrize("r,group,T,dtype", [(16, 4, 256, FP16), (8, 1, 33, FP16), (32, 2, 100, BF16), (64, 4, 70, FP16),
                                             (16, 2, 5, BF16), (64, 1, 9, BF16)])
def test_add_lora_bgmv_multi_vs_oracle(r, group, T, dtype):
    """q, k, v of one layer in one call pair on the reference layout, in place: three pools, projections of different
    widths, indices that repeat (grouped items) and some outside the pool, accumulate and delta forms."""
    from mlora import add_lora_bgmv_multi, plan_decode_ref
    rng = np.random.default_rng(r * 1000 + T)
    N, L, layer, scale = 11, 3, 2, 0.5
    shapes = [(512, 512), (512, 264), (1032, 2056)]            # q, k (narrower, tensor-parallel style), an odd-width pair
    was = [bits_of((rng.standard_normal((N, L, r, hin)) * 0.05).astype(np.float32), dtype) for hin, _ in shapes]
    wbs = [bits_of((rng.standard_normal((N, L, hout, r)) * 0.05).astype(np.float32), dtype) for _, hout in shapes]
    idx = rng.integers(0, N, T).astype(np.int64)
    idx[rng.random(T) < 0.4] = 3                                  # a hot adapter: several grouped items
    bad = np.zeros(T, bool)
    bad[::13] = True
    idx_dev = idx.copy()
    idx_dev[bad] = np.where(np.arange(T)[bad] % 2 == 0, -1, N + 2)
    xs = [bits_of(rng.standard_normal((T, hin)).astype(np.float32), dtype) for hin, _ in shapes]
    y0 = [bits_of(rng.standard_normal((T, hout)).astype(np.float32), dtype) for _, hout in shapes]
    ids = torch.from_numpy(idx_dev).cuda()
    plan = plan_decode_ref(ids, N, L, r, group=group)
    wa_t = [bits_to_torch(w, dtype, "cuda") for w in was]
    wb_t = [bits_to_torch(w, dtype, "cuda") for w in wbs]
    x_t = [bits_to_torch(x, dtype, "cuda") for x in xs]
    for accumulate in (True, False):
        ys = [bits_to_torch(y, dtype, "cuda") if accumulate else
              torch.full(y.shape, float("nan"), dtype=wa_t[0].dtype, device="cuda") for y in y0]
        say(f"add_lora_bgmv_multi r={r} group={group} T={T} accumulate={accumulate}")
        add_lora_bgmv_multi(ys, x_t, wa_t, wb_t, plan, layer, scale, accumulate=accumulate)
        torch.cuda.synchronize()
        for p in range(3):
            base = y0[p].copy() if accumulate else np.zeros_like(y0[p])
            want = base.copy()
            orc.add_lora_bgmv_ref(want, xs[p], was[p], wbs[p], idx, layer, scale, dtype)
            want[bad] = base[bad]                                  # an index outside the pool: no adapter
            got = torch_to_bits(ys[p])
            assert np.array_equal(got[bad], base[bad])
            assert_close_bits(got, want, dtype, f"projection {p}")


def test_add_lora_bgmv_multi_integer_inputs_bit_exact():
    from mlora import add_lora_bgmv_multi, plan_decode_ref
    rng = np.random.default_rng(77)
    N, L, r, H, T = 6, 2, 16, 512, 45
    wa = bits_of(rng.integers(-1, 2, (N, L, r, H)).astype(np.float32), FP16)
    wb = bits_of(rng.integers(-1, 2, (N, L, H, r)).astype(np.float32), FP16)
    idx = rng.integers(0, N, T).astype(np.int64)
    x = bits_of((rng.integers(-2, 3, (T, H)) * (rng.random((T, H)) < 0.05)).astype(np.float32), FP16)
    y0 = bits_of(rng.integers(-8, 9, (T, H)).astype(np.float32), FP16)
    want = y0.copy()
    orc.add_lora_bgmv_ref(want, x, wa, wb, idx, 1, 2.0, FP16)
    assert np.abs(f32_of(want, FP16)).max() < 2048
    plan = plan_decode_ref(torch.from_numpy(idx).cuda(), N, L, r, group=4)
    y = bits_to_torch(y0, FP16, "cuda")
    say("add_lora_bgmv_multi integer-valued inputs")
    add_lora_bgmv_multi([y], [bits_to_torch(x, FP16, "cuda")], [bits_to_torch(wa, FP16, "cuda")], [bits_to_torch(wb, FP16, "cuda")],
                        plan, 1, 2.0)
    torch.cuda.synchronize()
    assert np.array_equal(torch_to_bits(y), want)


def test_lora_gpu_qkv_in_one_call_pair_and_served_to_the_three_calls():
    """invoke_one_layer_qkv against the fp32 expression; the reference's q, k, v calls on one input get the same bits,
    computed once; a changed input, layer or weight set is computed afresh."""
    cfg = dict(n_layers=3, batch_size=20, lora_rank=16, hidden_dim=1024, tp_degree=2, max_prefill_batch_size=2)
    g = Lora_GPU(cfg, seed=5)
    x = torch.randn(37 % 20 + 1, 1024, device="cuda", dtype=torch.float16)
    bsz = x.shape[0]
    ids = torch.randint(0, 20, (bsz,), device="cuda", dtype=torch.int32)
    say("Lora_GPU.invoke_one_layer_qkv")
    q, k, v = g.invoke_one_layer_qkv(x, 2, lora_ids=ids)
    for name, got in zip("qkv", (q, k, v)):
        down, up = getattr(g, f"{name}_down"), getattr(g, f"{name}_up")
        want = torch.stack([x[i].float() @ down[ids[i], 2].float().t() @ up[ids[i], 2].float().t() for i in range(bsz)])
        assert got.shape == (bsz, 512) and torch.allclose(got.float(), want, rtol=RTOL, atol=ATOL)
    q1 = g.invoke_one_layer_q(x, 2, False, lora_ids=ids)
    plan_after_q = g._plan_gen
    k1 = g.invoke_one_layer_k(x, 2, False, lora_ids=ids)
    v1 = g.invoke_one_layer_v(x, 2, False, lora_ids=ids)
    assert g._plan_gen == plan_after_q                        # one plan, made before
    assert torch.equal(q1, q) and torch.equal(k1, k) and torch.equal(v1, v)
    x.mul_(2.0)                                                # same storage, new contents
    q2 = g.invoke_one_layer_q(x, 2, False, lora_ids=ids)
    assert not torch.equal(q2, q)
    g.merge_lora_prefill(0)                                    # weights may have changed: nothing stale is served
    k2 = g.invoke_one_layer_k(x, 2, False, lora_ids=ids)
    want = torch.stack([x[i].float() @ g.k_down[ids[i], 2].float().t() @ g.k_up[ids[i], 2].float().t() for i in range(bsz)])
    assert torch.allclose(k2.float(), want, rtol=RTOL, atol=ATOL)


def test_lora_gpu_fresh_index_tensor_every_step():
    """A serving loop builds lora_ids afresh each step (pre_process.py:50,100); a freed tensor's address is handed to
    the next one of the same size.  Every step must be computed from its own ids; in-place edits through torch and
    weight writes are seen as well."""
    cfg = dict(n_layers=2, batch_size=16, lora_rank=16, hidden_dim=512, tp_degree=1, max_prefill_batch_size=2)
    g = Lora_GPU(cfg, seed=9)
    bsz = 13
    x = torch.randn(bsz, 512, device="cuda", dtype=torch.float16)

    def want_of(name, ids, layer):
        down, up = getattr(g, f"{name}_down"), getattr(g, f"{name}_up")
        return torch.stack([x[i].float() @ down[ids[i], layer].float().t() @ up[ids[i], layer].float().t() for i in range(bsz)])

    rng = np.random.default_rng(21)
    addresses = set()
    say("Lora_GPU: fresh int32 lora_ids per step")
    for step in range(6):
        host = rng.integers(0, 16, bsz).tolist()
        ids = torch.tensor(host, dtype=torch.int32, device="cuda")     # as pre_process.py:100 makes them
        addresses.add(ids.data_ptr())
        for layer in range(2):
            for name in "qkv":
                got = getattr(g, f"invoke_one_layer_{name}")(x, layer, False, lora_ids=ids)
                assert torch.allclose(got.float(), want_of(name, host, layer), rtol=RTOL, atol=ATOL), (step, layer, name)
        del ids                                                         # the next step's tensor may reuse the address
    assert len(addresses) < 6, "the allocator never reused an address: the case this test is about did not occur"
    # the same tensor object edited in place through torch
    ids = torch.tensor(rng.integers(0, 16, bsz).tolist(), dtype=torch.int32, device="cuda")
    g.invoke_one_layer_q(x, 0, False, lora_ids=ids)
    ids.copy_(torch.tensor(host, dtype=torch.int32, device="cuda"))
    got = g.invoke_one_layer_q(x, 0, False, lora_ids=ids)
    assert torch.allclose(got.float(), want_of("q", host, 0), rtol=RTOL, atol=ATOL)
    # weights written in place between the q call and the k call of one layer
    g.k_down[host[0], 0].mul_(-3.0)
    got = g.invoke_one_layer_k(x, 0, False, lora_ids=ids)
    assert torch.allclose(got.float(), want_of("k", host, 0), rtol=RTOL, atol=ATOL)


def test_add_lora_bgmv_bad_index_leaves_row_untouched():
    rng = np.random.default_rng(3)
    N, L, r, H, T = 4, 1, 8, 128, 6
    wa = torch.randn(N, L, r, H, device="cuda", dtype=torch.float16)
    wb = torch.randn(N, L, H, r, device="cuda", dtype=torch.float16)
    x = torch.randn(T, H, device="cuda", dtype=torch.float16)
    y0 = torch.randn(T, H, device="cuda", dtype=torch.float16)
    idx = torch.tensor([0, 4, 1, -1, 31, 3], device="cuda")     # 4, -1, 31 are outside the pool
    y = y0.clone()
    say("add_lora_bgmv with out-of-range indices")
    add_lora_bgmv(y, x, wa, wb, idx, 0, 1.0)
    torch.cuda.synchronize()
    bad = torch.tensor([False, True, False, True, True, False], device="cuda")
    assert torch.equal(y[bad], y0[bad])
    assert not torch.equal(y[~bad], y0[~bad])


@pytest.mark.parametrize("B,Lpad,L,r,hin,hout,layer,dtype", [
    (3, 64, 2, 64, 4096, 4096, 1, FP16),
    (4, 37, 3, 16, 512, 768, 2, BF16),
    (1, 130, 1, 8, 256, 256, 0, FP16),
])
def test_prefill_ref_vs_oracle(B, Lpad, L, r, hin, hout, layer, dtype):
    rng = np.random.default_rng(B * 10 + r)
    A_T = bits_of((rng.standard_normal((B + 1, L, r, hin)) * 0.02).astype(np.float32), dtype)
    B_T = bits_of((rng.standard_normal((B + 1, L, hout, r)) * 0.02).astype(np.float32), dtype)
    x = bits_of(rng.standard_normal((B, Lpad, hin)).astype(np.float32), dtype)
    want = orc.prefill_bmm_ref(x, A_T[:B], B_T[:B], layer, dtype, round_mid=False)
    say(f"prefill ref B={B} Lpad={Lpad} r={r} {hin}x{hout}")
    y = lora_prefill_ref(bits_to_torch(x, dtype, "cuda"), bits_to_torch(A_T, dtype, "cuda"),
                         bits_to_torch(B_T, dtype, "cuda"), layer)
    torch.cuda.synchronize()
    assert_close_bits(torch_to_bits(y), want, dtype)


def test_lora_gpu_mirror_calls():
    """The calls LlamaTransformerLayerInfer._get_qkv makes (transformer_layer_infer.py:76-81,101-111)."""
    cfg = dict(n_layers=2, batch_size=12, lora_rank=16, hidden_dim=1024, tp_degree=1, max_prefill_batch_size=3,
               mode=["aaas-cached"])
    say("Lora_GPU mirror: decode and prefill through invoke_one_layer_{q,k,v}")
    g = Lora_GPU(cfg)
    assert g.q_down.shape == (12, 2, 16, 1024) and g.q_up.shape == (12, 2, 1024, 16)
    x = torch.randn(5, 1024, device="cuda", dtype=torch.float16)
    for name in "qkv":
        y = getattr(g, f"invoke_one_layer_{name}")(x, 1, False)
        inds = g.select_inds[4]
        down, up = getattr(g, f"{name}_down"), getattr(g, f"{name}_up")
        want = torch.stack([x[i].float() @ down[inds[i], 1].float().t() @ up[inds[i], 1].float().t() for i in range(5)])
        assert y.shape == (5, 1024) and torch.allclose(y.float(), want, rtol=RTOL, atol=ATOL)
    # the request's own adapter slots (infer_state.lora_ids, int32 as pre_process.py:100 builds them)
    ids = torch.tensor([11, 0, 7, 7, 3], dtype=torch.int32, device="cuda")
    y = g.invoke_one_layer_q(x, 0, False, lora_ids=ids)
    want = torch.stack([x[i].float() @ g.q_down[ids[i], 0].float().t() @ g.q_up[ids[i], 0].float().t() for i in range(5)])
    assert torch.allclose(y.float(), want, rtol=RTOL, atol=ATOL)
    xp = torch.randn(3, 20, 1024, device="cuda", dtype=torch.float16)
    for name in "qkv":
        y = getattr(g, f"invoke_one_layer_{name}")(xp, 0, True)
        down, up = getattr(g, f"{name}_down_prefill"), getattr(g, f"{name}_up_prefill")
        want = torch.bmm(torch.bmm(xp.float(), down[:3, 0].float().transpose(-1, -2)), up[:3, 0].float().transpose(-1, -2))
        assert y.shape == (3, 20, 1024) and torch.allclose(y.float(), want, rtol=RTOL, atol=ATOL)
    g.merge_lora_prefill(2, re_inds=[7, 3])
    assert torch.equal(g.k_up[7], g.k_up_prefill[0]) and torch.equal(g.v_down[3], g.v_down_prefill[1])
