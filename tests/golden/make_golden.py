"""Writes the committed fixtures under tests/golden/ from the CPU oracle.

    python tests/golden/make_golden.py

config1.json — configuration 1 (1 layer, K and V planes of 1024 pages x 16 tokens x 2 heads x 64
fp16, N(0,1) from numpy PCG64 seed 0): the gather ids, the scatter ids, and SHA-256 digests of the
pool, of the gathered staging buffer and of the pool after the scatter. The three oracle statements
(C, numpy, per-byte loops) must agree before anything is written.

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
    print("wrote config1.json, reference_scenarios.json")


if __name__ == "__main__":
    main()
