"""Seeded synthetic workloads of the benchmark configurations (adapter popularity, pool
contents, activations).  Index draws are made on the host with numpy so that a CPU checker
and the GPU see identical values; weights and activations are drawn by torch and can be
copied back for checking.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Tuple

import numpy as np
import torch

from .pool import AdapterPool

LLAMA7B_ATTN = {"q": (4096, 4096), "k": (4096, 4096), "v": (4096, 4096), "o": (4096, 4096)}
LLAMA7B_ALL = dict(LLAMA7B_ATTN, gate=(4096, 11008), up=(4096, 11008), down=(11008, 4096))
LLAMA13B_ALL = {"q": (5120, 5120), "k": (5120, 5120), "v": (5120, 5120), "o": (5120, 5120),
                "gate": (5120, 13824), "up": (5120, 13824), "down": (13824, 5120)}


def zipf_adapters(rng: np.random.Generator, n_tokens: int, n_adapters: int, alpha: float) -> np.ndarray:
    """Adapter id per token: popularity rank k drawn with p_k ~ k^-alpha, ranks mapped to
    adapter ids by a random permutation."""
    p = np.arange(1, n_adapters + 1, dtype=np.float64) ** (-alpha)
    p /= p.sum()
    ranks = rng.choice(n_adapters, size=n_tokens, p=p)
    return rng.permutation(n_adapters)[ranks].astype(np.int32)


def draw_lora_ids(popularity: np.ndarray, n_requests: int, seed: int = 0) -> np.ndarray:
    """Adapter id per request the way the reference's load generator draws it
    (``benchmark/client_maf.py:41-42,53``: ``np.random.seed(0)``, then one
    ``np.random.choice(total_lora_num, p=lora_popular)`` per request): the i-th value returned is
    the id of the i-th request that client sends."""
    popularity = np.asarray(popularity, np.float64)
    rs = np.random.RandomState(seed)
    return np.array([rs.choice(len(popularity), p=popularity) for _ in range(n_requests)], np.int32)


@dataclass
class Workload:
    name: str
    pool: AdapterPool
    tok_adapter: np.ndarray                      # int32 [T]
    ranks: np.ndarray                            # int32 [N]
    projections: Dict[str, Tuple[int, int]]
    n_layers: int


def fill_pool(pool: AdapterPool, ranks: np.ndarray, scalings: np.ndarray, rng: np.random.Generator,
              std: float = 0.02, shuffle_pages: bool = True, seed: int = 0) -> None:
    """Allocate every adapter (pages scattered when shuffle_pages) and fill all slabs with N(0, std)."""
    order = rng.permutation(pool.n_pages) if shuffle_pages else np.arange(pool.n_pages)
    pos = 0
    for slot, (r, s) in enumerate(zip(ranks, scalings)):
        need = (int(r) + pool.page_rows - 1) // pool.page_rows
        pool.allocate(slot, int(r), float(s), pages=[int(p) for p in order[pos:pos + need]])
        pos += need
    gen = torch.Generator(device=pool.device)
    gen.manual_seed(seed)
    for rows in list(pool.a_rows.values()) + list(pool.b_rows.values()):
        for layer in range(rows.shape[0]):
            # fp32 draw rounded to the pool dtype, one layer at a time to bound the transient
            rows[layer].copy_(torch.randn(rows[layer].shape, device=pool.device, dtype=torch.float32, generator=gen) * std)
    pool.sync()


def make_decode(name: str, projections: Dict[str, Tuple[int, int]], n_layers: int, n_tokens: int,
                n_adapters: int, ranks, alpha: float, seed: int, dtype=torch.float16, device="cuda",
                alpha_lora: float = 32.0, page_rows: int = 8, tok_adapter=None) -> Workload:
    rng = np.random.default_rng(seed)
    ranks = np.asarray(ranks, np.int32)
    if ranks.size == 1:
        ranks = np.full(n_adapters, int(ranks[0]), np.int32)
    n_pages = int(sum((int(r) + page_rows - 1) // page_rows for r in ranks))
    pool = AdapterPool(n_layers, projections, n_adapters, n_pages, page_rows=page_rows,
                       max_rank=int(ranks.max()), dtype=dtype, device=device)
    fill_pool(pool, ranks, alpha_lora / ranks.astype(np.float32), rng, seed=seed)
    tok = zipf_adapters(rng, n_tokens, n_adapters, alpha) if tok_adapter is None else np.asarray(tok_adapter, np.int32)
    return Workload(name, pool, tok, ranks, dict(projections), n_layers)


def config2(n_layers: int = 32, device="cuda") -> Workload:
    """Decode BGMV: Llama-7B q/k/v/o, 256 tokens, 64 rank-16 adapters, Zipf(1.0), fp16, scaling 2.0."""
    return make_decode("C2", LLAMA7B_ATTN, n_layers, 256, 64, [16], 1.0, seed=1002, device=device)


def config3(n_layers: int = 1, device="cuda") -> Workload:
    """Heterogeneous-rank decode: 128 adapters with ranks from {8,16,32,64}, all 7 projections, 128 tokens, Zipf(1.2)."""
    rng = np.random.default_rng(1003)
    ranks = rng.choice([8, 16, 32, 64], size=128).astype(np.int32)
    return make_decode("C3", LLAMA7B_ALL, n_layers, 128, 128, ranks, 1.2, seed=1003, device=device)
