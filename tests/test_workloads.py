"""Workload generators: the reference's adapter-popularity vectors (data fixtures copied from
benchmark/maf_lora_popularity/) and the per-request adapter draw of its load generator."""
import os

import numpy as np
import pytest

from mlora import workloads

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


@pytest.mark.parametrize("n", [128, 256, 512])
def test_popularity_vectors_are_probability_vectors(n):
    p = np.load(os.path.join(GOLDEN, f"maf_popularity_{n}.npy"), allow_pickle=False)
    assert p.shape == (n,) and p.dtype == np.float64
    assert np.all(p > 0) and abs(p.sum() - 1.0) < 1e-12
    # heavy head: the most popular eighth of the adapters carries about 78 % of the requests
    assert 0.75 < np.sort(p)[::-1][:n // 8].sum() < 0.82


def test_draw_lora_ids_follows_the_clients_stream():
    """benchmark/client_maf.py:41-42,53: np.random.seed(0) once, then np.random.choice(N, p=pop) per request.
    The legacy global generator seeded with 0 and drawing one id at a time is that stream."""
    p = np.load(os.path.join(GOLDEN, "maf_popularity_128.npy"), allow_pickle=False)
    ids = workloads.draw_lora_ids(p, 300, seed=0)
    state = np.random.get_state()
    try:
        np.random.seed(0)
        want = [np.random.choice(len(p), p=p) for _ in range(300)]
    finally:
        np.random.set_state(state)
    assert ids.dtype == np.int32 and ids.tolist() == want
    # and it follows the popularity: empirical frequencies of a long draw agree with p
    many = workloads.draw_lora_ids(p, 20000, seed=1)
    freq = np.bincount(many, minlength=len(p)) / len(many)
    top = np.argsort(p)[::-1][:5]
    assert np.allclose(freq[top], p[top], atol=0.01)


def test_zipf_adapters_range_and_skew():
    rng = np.random.default_rng(0)
    a = workloads.zipf_adapters(rng, 5000, 64, 1.0)
    assert a.dtype == np.int32 and a.min() >= 0 and a.max() < 64
    counts = np.sort(np.bincount(a, minlength=64))[::-1]
    assert counts[0] > 4 * counts[16]          # p_1 / p_17 = 17 under Zipf(1.0)


def test_decode_form_follows_the_batch_size():
    from mlora import ops
    assert [ops.default_group(t) for t in (1, 32, 64, 65, 128, 129, 256, 4096)] == [1, 1, 1, 2, 2, 4, 4, 4]
    # one work item per workgroup, one workgroup per compute unit: fused while that holds
    assert ops.decode_fused(64, 1, 3, 16) and ops.decode_fused(64, 1, 4, 16) and not ops.decode_fused(64, 1, 5, 16)
    assert ops.decode_fused(128, 2, 3, 32) and not ops.decode_fused(192, 2, 3, 48)
    assert not ops.decode_fused(128, 2, 3, 128)          # every token its own adapter: 128 items per projection
    assert not ops.decode_fused(8, 4, 1, 8) and not ops.decode_fused(8, 8, 1, 8)


def test_group_follows_the_launch_form_when_the_caller_names_its_projections():
    from mlora import ops
    # 128 tokens: three projections still run fused (2 tokens per item), seven run as the shrink + expand pair (4)
    assert ops.group_for(128, 3, 32) == 2 and ops.group_for(128, 7, 128) == 4
    # at 64 tokens and below the batch-size rule stands whatever the form; beyond 128 it is 4 anyway
    assert ops.group_for(64, 7, 16) == 1 and ops.group_for(32, 1, 8) == 1
    assert ops.group_for(256, 4, 64) == 4 and ops.group_for(512, 7, 1000) == 4
