"""Seeded synthetic workloads for the page-copy path: pool shapes and per-request page lists.

Page lists have the properties the reference's page managers give them
(Bi-KV/DistributedStorage/PageManager.py:20-49,105-115): ceil(tokens/page_size) ids per item, ids
unique within the manager, unordered (popped from a set), never contiguous by construction.
Everything is numpy with an explicit seed, so tests, the benchmark and the CPU baseline see the same
request streams.
"""
from dataclasses import dataclass, replace
from typing import Dict, List

import numpy as np


@dataclass(frozen=True)
class KVShape:
    name: str
    layers: int
    kv_heads: int
    head_dim: int
    page_tokens: int
    n_pages: int
    dtype: str            # "fp16" | "bf16" | "fp8"
    scales: bool = False  # fp32 scale per (page, layer, head, K/V)

    @property
    def elem_bytes(self) -> int:
        return 1 if self.dtype == "fp8" else 2

    @property
    def n_planes(self) -> int:
        return self.layers * 2

    @property
    def tile_bytes(self) -> int:
        return self.page_tokens * self.kv_heads * self.head_dim * self.elem_bytes

    @property
    def scale_tile_bytes(self) -> int:
        return self.kv_heads * 4 if self.scales else 0

    @property
    def page_bytes(self) -> int:
        """All layers, K and V, payload and scales of one logical page."""
        return (self.tile_bytes + self.scale_tile_bytes) * self.n_planes

    @property
    def pool_bytes(self) -> int:
        return self.page_bytes * self.n_pages

    def scaled(self, n_pages: int) -> "KVShape":
        """The same shape with a smaller pool (for CPU-sized tests)."""
        return replace(self, n_pages=n_pages)


SHAPES: Dict[str, KVShape] = {
    "tiny": KVShape("tiny", 1, 2, 64, 16, 1024, "fp16"),
    "qwen2_1p5b": KVShape("qwen2_1p5b", 28, 2, 128, 16, 65536, "bf16"),
    "qwen2_7b": KVShape("qwen2_7b", 28, 4, 128, 16, 131072, "bf16"),
    "llama3_8b": KVShape("llama3_8b", 32, 8, 128, 32, 32768, "fp16"),
    "llama3_70b_fp8": KVShape("llama3_70b_fp8", 80, 8, 128, 16, 49152, "fp8", scales=True),
}


def _pages_for(tokens: np.ndarray, page_tokens: int) -> np.ndarray:
    return (tokens + page_tokens - 1) // page_tokens


def _split(ids: np.ndarray, counts: np.ndarray) -> List[np.ndarray]:
    cuts = np.cumsum(counts)[:-1]
    return [np.ascontiguousarray(a) for a in np.split(ids, cuts)]


def _fit(counts: np.ndarray, budget: int) -> np.ndarray:
    """Shrinks request sizes proportionally (at least one page each) until they fit `budget` pages."""
    counts = counts.copy()
    while counts.sum() > budget:
        over = counts.sum() - budget
        big = counts > 1
        if not big.any():
            raise ValueError("pool too small for this many requests")
        take = np.minimum(counts[big] - 1, np.maximum(1, (counts[big] * over) // counts[big].sum() + 1))
        counts[big] -= take
    return counts


def tiny(shape: KVShape = SHAPES["tiny"], n_ids: int = 64, seed: int = 0):
    """Config 1: gather `n_ids` unique random pages, scatter them back to a different random set."""
    g = np.random.default_rng(seed).permutation(shape.n_pages)[:n_ids].astype(np.int64)
    s = np.random.default_rng(seed + 1).permutation(shape.n_pages)[:n_ids].astype(np.int64)
    return {"gather": [g], "scatter": [s]}


def uniform_requests(shape: KVShape, n_requests: int, lo_tokens: int, hi_tokens: int, seed: int):
    """Config 2: lengths uniform in [lo, hi] tokens; pages are consecutive slices of one random
    permutation of the pool (every id used at most once)."""
    rng = np.random.default_rng(seed)
    tokens = rng.integers(lo_tokens, hi_tokens + 1, size=n_requests)
    counts = _fit(_pages_for(tokens, shape.page_tokens), shape.n_pages)
    perm = rng.permutation(shape.n_pages).astype(np.int64)
    return {"gather": _split(perm[: counts.sum()], counts)}


def mixed_gather_scatter(shape: KVShape, n_requests: int, lo_tokens: int, hi_tokens: int, seed: int,
                         dup_fraction: float = 0.10):
    """Config 3: the first half of the requests gather, the second half scatter into freshly
    allocated page ids. About `dup_fraction` of the gather ids are overwritten with ids taken from
    OTHER gather requests (shared prefixes -> duplicate reads). Scatter ids are unique and disjoint
    from the gather ids."""
    rng = np.random.default_rng(seed)
    tokens = rng.integers(lo_tokens, hi_tokens + 1, size=n_requests)
    counts = _fit(_pages_for(tokens, shape.page_tokens), shape.n_pages)
    perm = rng.permutation(shape.n_pages).astype(np.int64)
    half = n_requests // 2
    g_counts, s_counts = counts[:half], counts[half:]
    g_ids = perm[: g_counts.sum()].copy()
    s_ids = perm[g_counts.sum(): g_counts.sum() + s_counts.sum()]
    n_g = len(g_ids)
    owner = np.repeat(np.arange(half), g_counts)
    n_dup = int(round(dup_fraction * n_g))
    if n_dup and half > 1:
        where = rng.choice(n_g, size=n_dup, replace=False)
        donors = rng.integers(0, n_g, size=n_dup)
        # a donor must belong to another request; step forward until it does
        for k in range(n_dup):
            d = donors[k]
            while owner[d] == owner[where[k]]:
                d = (d + 1) % n_g
            donors[k] = d
        snapshot = g_ids.copy()
        g_ids[where] = snapshot[donors]
    return {"gather": _split(g_ids, g_counts), "scatter": _split(s_ids, s_counts)}


def lognormal_requests(shape: KVShape, n_requests: int, median_tokens: int, max_tokens: int, seed: int,
                       sigma: float = 1.0):
    """Config 4: lengths log-normal (median `median_tokens`), clipped to [page_tokens, max_tokens].
    Each request draws its ids from its own random permutation of the pool (requests are staged one
    after the other, so ids may repeat across requests)."""
    rng = np.random.default_rng(seed)
    tokens = np.rint(rng.lognormal(np.log(median_tokens), sigma, size=n_requests)).astype(np.int64)
    tokens = np.clip(tokens, shape.page_tokens, max_tokens)
    counts = np.minimum(_pages_for(tokens, shape.page_tokens), shape.n_pages)
    return {"gather": [rng.permutation(shape.n_pages)[:c].astype(np.int64) for c in counts]}


def zipf_requests(shape: KVShape, n_requests: int, lo_tokens: int, hi_tokens: int, seed: int,
                  exponent: float = 1.1):
    """Config 5: lengths ~ k^-exponent on [lo, hi] tokens (many single-page requests, a few huge).
    Gather ids come from one permutation that is cycled when exhausted (duplicates across requests
    are legal reads); scatter ids are a unique slice of a second permutation, for as many leading
    requests as fit the pool."""
    rng = np.random.default_rng(seed)
    k = np.arange(lo_tokens, hi_tokens + 1, dtype=np.float64)
    p = k ** (-exponent)
    p /= p.sum()
    tokens = rng.choice(np.arange(lo_tokens, hi_tokens + 1), size=n_requests, p=p)
    counts = np.minimum(_pages_for(tokens, shape.page_tokens), shape.n_pages)
    total = int(counts.sum())
    perm = rng.permutation(shape.n_pages).astype(np.int64)
    g_ids = np.resize(perm, total)
    perm2 = rng.permutation(shape.n_pages).astype(np.int64)
    fits = np.cumsum(counts) <= shape.n_pages
    n_fit = int(fits.sum())
    s_counts = counts[:n_fit]
    return {"gather": _split(g_ids, counts),
            "scatter": _split(perm2[: s_counts.sum()], s_counts) if n_fit else []}


def named(name: str, shape: KVShape = None):
    """The request streams of the five named configurations (seeds 0, 2, 3, 4, 5)."""
    shape = shape or SHAPES[name]
    if name == "tiny":
        return tiny(shape, 64, seed=0)
    if name == "qwen2_1p5b":
        return uniform_requests(shape, 32, 512, 4096, seed=2)
    if name == "qwen2_7b":
        return mixed_gather_scatter(shape, 64, 1024, 8192, seed=3)
    if name == "llama3_8b":
        return lognormal_requests(shape, 128, 2048, 16384, seed=4)
    if name == "llama3_70b_fp8":
        return zipf_requests(shape, 256, 16, 32768, seed=5)
    raise KeyError(name)
