"""Writes the committed fixtures under tests/golden/ from the CPU oracle.

    python tests/golden/make_golden.py

config1.json — configuration 1 (1 layer, K and V planes of 1024 pages x 16 tokens x 2 heads x 64
fp16, N(0,1) from numpy PCG64 seed 0): the gather ids, the scatter ids, and SHA-256 digests of the
pool, of the gathered staging buffer and of the pool after the scatter. The three oracle statements
(C, numpy, per-byte loops) must agree before anything is written.

packed_and_layout.json — SHA-256 digests of a seeded packed (token-exact) transfer and of a seeded
layout change (both pool forms): inputs, the tensor the consumer receives, the layers after a load
and the token-major buffer after a store.

reference_scenarios.json — the parameters and expected results of the only two known-answer
scenarios the reference holds for this path (Bi-KV/SharedMemory/CUDA_Shared/test_page_ipc.py:
41-65,127-150 and test_zero_copy.py:30-48,86-103). These are data read from those scripts.
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [ROOT, os.path.join(ROOT, "bi-kv_amd")]

from bikv_pagecopy import workloads  # noqa: E402  (request streams are shared with the product)
from oracle import pagecopy_oracle as oracle  # noqa: E402


def sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def config1_pool():
    shape = workloads.SHAPES["tiny"]
    rng = np.random.default_rng(0)
    return rng.standard_normal((shape.n_planes, shape.n_pages, shape.tile_bytes // 2)).astype(np.float16)


def packed_case():
    """Seeded inputs of the packed (token-exact) transfer fixture."""
    rng = np.random.default_rng(101)
    page_size, ept, pool_pages = 16, 24, 64
    pool = rng.integers(0, 65536, size=(pool_pages * page_size, ept), dtype=np.uint16)
    pages_list = [[17, 3, 60], [9], [], [41, 42, 0, 5], [33]]
    tokens = [35, 16, 0, 64, 1]
    return pool, pages_list, tokens, page_size


def layout_case(form):
    """Seeded inputs of the layout-change fixture: token shape (32, 2, 4, 2) uint16, pages of 4 tokens."""
    rng = np.random.default_rng(102)
    P, D, H, L, blocks, n_tm = 4, 32, 2, 4, 9, 6
    tm = rng.integers(0, 65536, size=(n_tm, P, D, H, L, 2), dtype=np.uint16)
    shape = (blocks * P, 2, H, D) if form == "token_kv" else (blocks, 2, P, H, D)
    layers = [rng.integers(0, 65536, size=shape, dtype=np.uint16) for _ in range(L)]
    load = (np.array([7, 0, 3, 8], dtype=np.int64), np.array([5, 1, 0, 2], dtype=np.int64))
    store = (np.array([2, 8, 4], dtype=np.int64), np.array([3, 4, 0], dtype=np.int64))
    return tm, layers, load, store


def main():
    wl = workloads.named("tiny")
    pool = config1_pool()
    out = {"pool_sha256": sha(pool), "gather_ids": wl["gather"][0].tolist(),
           "scatter_ids": wl["scatter"][0].tolist()}
    for layout in ("layer_major", "page_major"):
        g_c = oracle.gather_layered_c(pool, wl["gather"], layout)
        g_np = oracle.gather_layered_np(pool, wl["gather"], layout)
        assert g_c.tobytes() == g_np.tobytes()
        small = [wl["gather"][0][:3]]
        assert oracle.gather_layered_loops(pool, small, layout).tobytes() == \
            oracle.gather_layered_np(pool, small, layout).tobytes()
        p2 = pool.copy()
        oracle.scatter_layered_c(p2, wl["scatter"], g_c, layout)
        p3 = pool.copy()
        oracle.scatter_layered_np(p3, wl["scatter"], g_np, layout)
        assert p2.tobytes() == p3.tobytes()
        out[layout] = {"staging_sha256": sha(g_c), "pool_after_scatter_sha256": sha(p2)}
    with open(os.path.join(HERE, "config1.json"), "w") as f:
        json.dump(out, f, indent=1)

    scenarios = {
        "test_page_ipc": {
            "source": "Bi-KV/SharedMemory/CUDA_Shared/test_page_ipc.py:41-65,127-150,171-176",
            "page_size": 50, "num_pages": 200, "head_size": 128, "num_kv_heads": 2, "num_layers": 28,
            "kv_pair": 2, "dtype": "float16", "fill_value": 7,
            "src_offsets": "i * page_elements", "dest_offsets": "i * page_elements",
            "buffer_size": 2 * 1024 ** 3, "num_transfers": 11,
            "expected_dim": 5, "expected_shape": [10000, 128, 2, 28, 2], "expected_value": 7,
        },
        "test_zero_copy": {
            "source": "Bi-KV/SharedMemory/CUDA_Shared/test_zero_copy.py:30-48,86-103,118-123",
            "page_size": 50, "num_pages": 200, "head_size": 128, "num_kv_heads": 2, "num_layers": 28,
            "kv_pair": 2, "dtype": "float16", "fill_value": 7,
            "page_indices": "arange(num_pages)  (element offsets, not scaled by page_elements)",
            "dest_offsets": "i * page_elements",
            "buffer_size": 2 * 1024 ** 3, "num_transfers": 11,
            "expected_shape": [10000, 128, 2, 28, 2], "expected_value": 7,
        },
    }
    with open(os.path.join(HERE, "reference_scenarios.json"), "w") as f:
        json.dump(scenarios, f, indent=1)

    # packed transfer and layout change: digests of seeded cases; two oracle statements must agree first
    more = {}
    pool, pages_list, tokens, page_size = packed_case()
    so, do, total = oracle.build_offsets_loops(pages_list, [(0, t) for t in tokens], page_size)
    sizes = []
    for pages, t in zip(pages_list, tokens):
        sizes += [page_size] * (len(pages) - 1) + ([t % page_size or page_size] if pages else [])
    dst = np.zeros((total, pool.shape[1]), dtype=np.uint16)
    assert oracle.copy_runs_ragged_c(pool, dst, so, do, sizes, page_size, unit_elems=pool.shape[1]) == 0
    assert dst.tobytes() == oracle.packed_items_np(pool, pages_list, tokens, page_size).tobytes()
    more["packed_transfer"] = {"pool_sha256": sha(pool), "total_tokens": int(total), "received_sha256": sha(dst)}
    for form in ("token_kv", "block_kv"):
        tm, layers, load, store = layout_case(form)
        a_layers, a_tm = [x.copy() for x in layers], tm.copy()
        b_layers, b_tm = [x.copy() for x in layers], tm.copy()
        assert oracle.transpose_pages_c(a_layers, form, a_tm, load[0], load[1], "load") == 0
        oracle.transpose_pages_np(b_layers, form, b_tm, load[0], load[1], "load")
        assert all(x.tobytes() == y.tobytes() for x, y in zip(a_layers, b_layers))
        after_load = sha(np.stack(a_layers))
        assert oracle.transpose_pages_c(a_layers, form, a_tm, store[0], store[1], "store") == 0
        oracle.transpose_pages_np(b_layers, form, b_tm, store[0], store[1], "store")
        assert a_tm.tobytes() == b_tm.tobytes()
        more[f"layout_change_{form}"] = {"tm_sha256": sha(tm), "layers_sha256": sha(np.stack(layers)),
                                         "layers_after_load_sha256": after_load, "tm_after_store_sha256": sha(a_tm)}
    with open(os.path.join(HERE, "packed_and_layout.json"), "w") as f:
        json.dump(more, f, indent=1)
    print("wrote config1.json, reference_scenarios.json")


if __name__ == "__main__":
    main()
