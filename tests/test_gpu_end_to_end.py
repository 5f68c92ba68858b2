"""The reference's whole transfer, both ways, in one process on one GPU, every step through this
library: cache pool (token-major, Bi-KV/DistributedStorage/kvcache.py:38-43) -> page copy into the
consumer's ring (kvcache.py:132-239) -> Worker receives the tensor (Worker/Worker.py:166-173) ->
pages land in the model's per-layer paged pool (Worker.py:74-78; the step the reference leaves out)
-> and back: pool blocks -> token-major pages -> ring -> the cache's pool pages chosen by its page
manager (DistributedStorage/PageManager.py:105-115). Expected bytes come from the oracle."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_cache_to_worker_and_back(lib, oracle, cuda):
    import bikv_pagecopy as bk
    import ipc_service as ipc
    from bikv_pagecopy import kvcache_calls
    print("[case] end to end: cache -> ring -> paged pool -> ring -> cache", flush=True)
    rng = np.random.default_rng(83)
    D, H, L, P = 64, 2, 4, 16                                  # token_shape (D, H, L, 2), pages of 16 tokens
    dims, ept = (D, H, L, 2), D * H * L * 2
    cache_pages, worker_blocks = 40, 24
    cache_h = rng.integers(0, 65536, size=(cache_pages * P, D, H, L, 2), dtype=np.uint16)
    cache_d = torch.from_numpy(cache_h.view(np.int16)).view(torch.float16).to(cuda)
    layers_h = [rng.integers(0, 65536, size=(worker_blocks * P, 2, H, D), dtype=np.uint16) for _ in range(L)]
    layers_d = [torch.from_numpy(a.view(np.int16)).view(torch.float16).to(cuda) for a in layers_h]
    kv = bk.NHDPool.from_token_kv_layers(layers_d, P)
    name = f"/bikv_test_e2e_{os.getpid()}"
    ipc.producer_cleanup()
    ipc.consumer_cleanup()
    ipc.consumer_init(0, name, 32 << 20)
    ipc.producer_init(0, name)
    idx = bk.RunIndexPool(max_pages=cache_pages, device=cuda)
    try:
        # ---- cache -> worker: two items of whole pages, ids out of order as a page manager hands them out
        pages_list = [[31, 4, 17], [9, 38]]
        info = {"infer_worker": 0, "token_num": 5 * P, "id_token_pair": [(100, 3 * P), (101, 2 * P)],
                "cache_pages_list": pages_list}
        n, tokens = kvcache_calls.shared_data_batch_pages(cache_d, info, P, dims, index_pool=idx)
        recv = ipc.consumer_receive(timeout_ms=5000)
        assert (n, tokens) == (5, 5 * P) and tuple(recv.shape) == (5 * P,) + dims
        blocks = np.array([20, 3, 11, 7, 0], dtype=np.int64)          # free blocks of the worker's pool
        kv.load_token_major(recv.view(5, P, D, H, L, 2), torch.from_numpy(blocks).to(cuda))
        kv.check()
        flat = [p for pages in pages_list for p in pages]
        tm_h = np.stack([cache_h[p * P:(p + 1) * P] for p in flat])   # what the ring must have held
        assert recv.cpu().contiguous().view(torch.int16).numpy().tobytes() == tm_h.tobytes()
        assert oracle.transpose_pages_c(layers_h, "token_kv", tm_h, blocks, np.arange(5), "load") == 0
        for l in range(L):
            assert layers_d[l].cpu().view(torch.int16).numpy().tobytes() == layers_h[l].tobytes(), f"layer {l}"

        # ---- worker -> cache: three other blocks go out token-major and land in cache pages 2, 25, 13
        out_blocks = np.array([5, 23, 14], dtype=np.int64)
        send = torch.empty((3, P, D, H, L, 2), dtype=torch.float16, device=cuda)
        kv.store_token_major(send, torch.from_numpy(out_blocks).to(cuda))
        kv.check()
        ipc.producer_send(send.view(3 * P, D, H, L, 2))
        back = ipc.consumer_receive(timeout_ms=5000)
        assert tuple(back.shape) == (3 * P, D, H, L, 2)
        dest_pages = np.array([2, 25, 13], dtype=np.int64)
        so = torch.arange(3, dtype=torch.int64, device=cuda) * (P * ept)
        do = torch.from_numpy(dest_pages * (P * ept)).to(cuda)
        bk.copy_runs(back, cache_d, so, do, P * ept)
        from bikv_pagecopy import runs
        runs.check(cuda)
        send_h = np.zeros((3, P, D, H, L, 2), dtype=np.uint16)
        assert oracle.transpose_pages_c(layers_h, "token_kv", send_h, out_blocks, np.arange(3), "store") == 0
        want = cache_h.copy()
        for i, p in enumerate(dest_pages):
            want[p * P:(p + 1) * P] = send_h[i]
        assert cache_d.cpu().view(torch.int16).numpy().tobytes() == want.tobytes()
    finally:
        ipc.producer_cleanup()
        ipc.consumer_cleanup()
        kv.close()
