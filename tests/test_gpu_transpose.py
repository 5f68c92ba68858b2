"""Fused page move + layout change (token-major pages <-> per-layer paged NHD pool) on a real GPU,
bit-exact against the oracle, through the C ABI."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

_NP = {1: np.uint8, 2: np.uint16, 4: np.uint32}
_TORCH = {1: torch.uint8, 2: torch.float16, 4: torch.float32}


def _to_np(t):
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()


def _make(rng, form, es, P, D, H, L, blocks, n_tm, cuda):
    dt = _NP[es]
    tm_h = rng.integers(0, np.iinfo(dt).max, size=(n_tm, P, D, H, L, 2), dtype=dt)
    shape = (blocks * P, 2, H, D) if form == "token_kv" else (blocks, 2, P, H, D)
    layers_h = [rng.integers(0, np.iinfo(dt).max, size=shape, dtype=dt) for _ in range(L)]
    tm_d = torch.from_numpy(tm_h.view(np.uint8)).to(cuda).view(_TORCH[es]).view(tm_h.shape)
    layers_d = [torch.from_numpy(a.view(np.uint8)).to(cuda).view(_TORCH[es]).view(a.shape) for a in layers_h]
    return tm_h, layers_h, tm_d, layers_d


@pytest.mark.parametrize("form", ["token_kv", "block_kv"])
@pytest.mark.parametrize("es,P,D,H,L", [
    (2, 16, 128, 2, 28),     # the reference's Qwen2-1.5B token shape (Model/qwen2.py:512-522), block of 16
    (2, 16, 128, 4, 28),     # Qwen2-7B
    (2, 32, 128, 8, 32),     # Llama-3-8B: 512 columns -> four column chunks per token
    (1, 16, 128, 8, 80),     # fp8 payload, 1280 columns
    (4, 4, 64, 2, 6),        # fp32
    (2, 3, 8, 2, 2),         # the smallest shape the kernel takes (one vector per row)
    (2, 5, 80, 4, 3),        # head_dim 80: 10 vectors per row, not a multiple of 4
    (2, 4, 96, 4, 5),        # head_dim 96: word-pair kernel with 12 vectors per compute row
    (2, 2, 32, 1, 4),        # the smallest shape of the word-pair kernel: one vector per token-major row
    (2, 3, 256, 2, 36),      # head_dim 256, 144 columns: the tile is cut into column chunks
    (1, 3, 64, 2, 4),        # 1-byte elements, the smallest pair-kernel shape (one vector per row)
    (4, 2, 16, 3, 2),        # 4-byte elements, head_dim 16
    (4, 3, 128, 4, 16),      # fp32, 128 columns: chunked
    (2, 4, 64, 4, 1),        # a single layer
    (2, 64, 128, 8, 32),     # 64 tokens per block x four column chunks: 256 workgroups per page
    (4, 3, 64, 2, 5),        # fp32 with half-KiB K rows and an odd layer count: the last wave's upper half-wave has no layer
    (1, 6, 128, 4, 6),       # 1-byte elements whose K rows are half a KiB (4 heads x 128)
])
@pytest.mark.parametrize("pairs", [1, 0])
def test_load_and_store_match_oracle(lib, oracle, cuda, form, es, P, D, H, L, pairs):
    import bikv_pagecopy as bk
    print(f"[case] layout change {form} es={es} P={P} D={D} H={H} L={L} pairs={pairs}", flush=True)
    bk.set_tuning(transpose_pairs=pairs)
    rng = np.random.default_rng(es * 1000 + D + H + L)
    blocks, n_tm = 9, 7
    tm_h, layers_h, tm_d, layers_d = _make(rng, form, es, P, D, H, L, blocks, n_tm, cuda)
    pool = (bk.NHDPool.from_token_kv_layers(layers_d, P) if form == "token_kv"
            else bk.NHDPool.from_block_kv_layers(layers_d))
    block_ids = rng.permutation(blocks)[:5].astype(np.int64)
    tm_pages = rng.permutation(n_tm)[:5].astype(np.int64)
    b_d, t_d = torch.from_numpy(block_ids).to(cuda), torch.from_numpy(tm_pages).to(cuda)
    # load: token-major pages -> pool blocks
    pool.load_token_major(tm_d, b_d, t_d)
    pool.check()
    assert oracle.transpose_pages_c(layers_h, form, tm_h, block_ids, tm_pages, "load") == 0
    for l in range(L):
        assert _to_np(layers_d[l]).tobytes() == layers_h[l].tobytes(), f"layer {l}"
    # store: other pool blocks -> other token-major pages
    block_ids2 = rng.permutation(blocks)[:4].astype(np.int64)
    tm_pages2 = rng.permutation(n_tm)[:4].astype(np.int64)
    pool.store_token_major(tm_d, torch.from_numpy(block_ids2).to(cuda), torch.from_numpy(tm_pages2).to(cuda))
    pool.check()
    bk.set_tuning(transpose_pairs=1)
    assert oracle.transpose_pages_c(layers_h, form, tm_h, block_ids2, tm_pages2, "store") == 0
    assert _to_np(tm_d).tobytes() == tm_h.tobytes()


@pytest.mark.parametrize("block", [128, 256, 1024])
def test_word_pair_kernel_at_other_workgroup_sizes(lib, oracle, cuda, block):
    import bikv_pagecopy as bk
    print(f"[case] layout change, word-pair kernel with {block} lanes", flush=True)
    rng = np.random.default_rng(block)
    P, D, H, L, blocks, n_tm = 5, 64, 3, 4, 8, 6
    tm_h, layers_h, tm_d, layers_d = _make(rng, "block_kv", 2, P, D, H, L, blocks, n_tm, cuda)
    pool = bk.NHDPool.from_block_kv_layers(layers_d)
    ids = rng.permutation(blocks)[:5].astype(np.int64)
    pages = rng.permutation(n_tm)[:5].astype(np.int64)
    bk.set_tuning(transpose_block=block)
    try:
        pool.load_token_major(tm_d, torch.from_numpy(ids).to(cuda), torch.from_numpy(pages).to(cuda))
        pool.check()
        oracle.transpose_pages_c(layers_h, "block_kv", tm_h, ids, pages, "load")
        for l in range(L):
            assert _to_np(layers_d[l]).tobytes() == layers_h[l].tobytes(), f"layer {l}"
        ids2 = rng.permutation(blocks)[:4].astype(np.int64)
        pages2 = rng.permutation(n_tm)[:4].astype(np.int64)
        pool.store_token_major(tm_d, torch.from_numpy(ids2).to(cuda), torch.from_numpy(pages2).to(cuda))
        pool.check()
        oracle.transpose_pages_c(layers_h, "block_kv", tm_h, ids2, pages2, "store")
        assert _to_np(tm_d).tobytes() == tm_h.tobytes()
    finally:
        bk.reset_tuning()


@pytest.mark.parametrize("kvswap", [1, 0])
@pytest.mark.parametrize("block", [0, 128, 256, 512, 1024])
def test_half_wave_exchange_on_the_workers_own_shape(lib, oracle, cuda, block, kvswap):
    """The Worker's tensors at 2 KV heads x 128 x fp16 (K and V rows of a token adjacent, half a KiB each):
    the pair kernel reads and writes whole KiB and exchanges half-waves; with the exchange switched off
    every lane addresses its own rows. Both, at every workgroup size, against the oracle."""
    import bikv_pagecopy as bk
    print(f"[case] layout change, half-wave exchange={kvswap}, {block or 'default'} lanes", flush=True)
    rng = np.random.default_rng(900 + block + kvswap)
    P, D, H, L, blocks, n_tm = 7, 128, 2, 10, 11, 8
    tm_h, layers_h, tm_d, layers_d = _make(rng, "token_kv", 2, P, D, H, L, blocks, n_tm, cuda)
    pool = bk.NHDPool.from_token_kv_layers(layers_d, P)
    bk.set_tuning(transpose_block=block, transpose_kvswap=kvswap)
    try:
        ids = rng.permutation(blocks)[:6].astype(np.int64)
        pages = rng.permutation(n_tm)[:6].astype(np.int64)
        pool.load_token_major(tm_d, torch.from_numpy(ids).to(cuda), torch.from_numpy(pages).to(cuda))
        pool.check()
        oracle.transpose_pages_c(layers_h, "token_kv", tm_h, ids, pages, "load")
        for l in range(L):
            assert _to_np(layers_d[l]).tobytes() == layers_h[l].tobytes(), f"layer {l}"
        ids2 = rng.permutation(blocks)[:5].astype(np.int64)
        pages2 = rng.permutation(n_tm)[:5].astype(np.int64)
        pool.store_token_major(tm_d, torch.from_numpy(ids2).to(cuda), torch.from_numpy(pages2).to(cuda))
        pool.check()
        oracle.transpose_pages_c(layers_h, "token_kv", tm_h, ids2, pages2, "store")
        assert _to_np(tm_d).tobytes() == tm_h.tobytes()
    finally:
        bk.reset_tuning()


def test_default_tm_pages_is_a_dense_received_buffer(lib, oracle, cuda):
    """A received tensor (tokens,)+token_shape (Worker.py:166-169) is pages 0..n-1 in order."""
    import bikv_pagecopy as bk
    print("[case] layout change dense buffer", flush=True)
    rng = np.random.default_rng(5)
    P, D, H, L, blocks = 16, 128, 2, 28, 12
    tm_h, layers_h, tm_d, layers_d = _make(rng, "token_kv", 2, P, D, H, L, blocks, 6, cuda)
    pool = bk.NHDPool.from_token_kv_layers(layers_d, P)
    ids = rng.permutation(blocks)[:6].astype(np.int64)
    recv = tm_d.view(6 * P, D, H, L, 2)                      # the reference's shape
    pool.load_token_major(recv, torch.from_numpy(ids).to(cuda))
    pool.check()
    oracle.transpose_pages_c(layers_h, "token_kv", tm_h, ids, np.arange(6), "load")
    for l in range(L):
        assert _to_np(layers_d[l]).tobytes() == layers_h[l].tobytes()
    # the model-side view of one element, spelled out
    t, d, h, l, k = 3, 77, 1, 20, 1
    assert layers_d[l][ids[2] * P + t, k, h, d].item() == recv[2 * P + t, d, h, l, k].item()


def test_page_list_walks_in_block_order_with_the_same_result(lib, oracle, cuda):
    """NHDPool.page_list sorts a host-built page list by block id and keeps each page with its block: the
    pool and the stored pages are byte for byte what the unsorted list gives."""
    import bikv_pagecopy as bk
    print("[case] layout change, sorted page list", flush=True)
    rng = np.random.default_rng(9)
    P, D, H, L, blocks, n = 16, 128, 2, 6, 40, 17
    tm_h, layers_h, tm_d, layers_d = _make(rng, "token_kv", 2, P, D, H, L, blocks, n, cuda)
    pool = bk.NHDPool.from_token_kv_layers(layers_d, P)
    ids = rng.permutation(blocks)[:n].astype(np.int64)
    tm_pages = rng.permutation(n).astype(np.int64)           # page i of the call is tm page tm_pages[i]
    b, p = pool.page_list(ids, tm_pages, sort=True, check_unique=True)
    assert bool((b[1:] > b[:-1]).all()) and sorted(b.tolist()) == sorted(ids.tolist())
    assert dict(zip(b.tolist(), p.tolist())) == dict(zip(ids.tolist(), tm_pages.tolist()))
    pool.load_token_major(tm_d, b, p)
    pool.check()
    oracle.transpose_pages_c(layers_h, "token_kv", tm_h, ids, tm_pages, "load")
    for l in range(L):
        assert _to_np(layers_d[l]).tobytes() == layers_h[l].tobytes()
    out = torch.zeros_like(tm_d)
    pool.store_token_major(out, b, p)
    pool.check()
    assert torch.equal(out.view(torch.int16), tm_d.view(torch.int16))
    # unsorted, default pages, and the duplicate check
    b2, p2 = pool.page_list(ids)
    assert b2.tolist() == ids.tolist() and p2.tolist() == list(range(n))
    with pytest.raises(RuntimeError, match="block ids: destination id"):
        pool.page_list([3, 5, 3], check_unique=True)


def test_bad_ids_are_skipped_and_reported_and_shapes_are_checked(lib, cuda):
    import bikv_pagecopy as bk
    print("[case] layout change error paths", flush=True)
    P, D, H, L, blocks = 4, 64, 2, 4, 5
    layers = [torch.zeros((blocks * P, 2, H, D), dtype=torch.float16, device=cuda) for _ in range(L)]
    pool = bk.NHDPool.from_token_kv_layers(layers, P)
    tm = torch.ones((3, P, D, H, L, 2), dtype=torch.float16, device=cuda)
    pool.load_token_major(tm, torch.tensor([1, 9, 2], device=cuda), torch.tensor([0, 1, 5], device=cuda))
    with pytest.raises(RuntimeError, match="page-id"):
        pool.check()
    assert torch.all(layers[0][1 * P:2 * P] == 1) and not layers[0][2 * P:3 * P].any()   # page 0 moved, others not
    with pytest.raises(RuntimeError, match="multiples of"):
        bk.NHDPool.from_token_kv_layers([torch.zeros((8, 2, 1, 12), dtype=torch.float16, device=cuda)], 4)
    with pytest.raises(RuntimeError, match="CUDA"):
        bk.NHDPool.from_token_kv_layers([torch.zeros((8, 2, 2, 64), dtype=torch.float16)], 4)
    with pytest.raises(RuntimeError, match="element size"):
        pool.load_token_major(tm.float(), torch.tensor([1], device=cuda))
    with pytest.raises(RuntimeError, match="int64"):
        pool.load_token_major(tm, torch.tensor([1], device=cuda, dtype=torch.int32))


@pytest.mark.parametrize("form", ["token_kv", "block_kv"])
def test_layout_change_against_committed_digests(lib, cuda, form):
    """The kernels against tests/golden/packed_and_layout.json directly (no oracle in the loop)."""
    import hashlib
    import importlib.util
    import json
    import os
    import bikv_pagecopy as bk
    print(f"[case] layout change golden digests {form}", flush=True)
    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(golden, "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    with open(os.path.join(golden, "packed_and_layout.json")) as f:
        e = json.load(f)[f"layout_change_{form}"]
    sha = lambda a: hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()
    tm, layers, load, store = mg.layout_case(form)
    tm_d = torch.from_numpy(tm.view(np.int16)).to(cuda).view(torch.float16)
    layers_d = [torch.from_numpy(a.view(np.int16)).to(cuda).view(torch.float16) for a in layers]
    P = tm.shape[1]
    pool = bk.NHDPool.from_token_kv_layers(layers_d, P) if form == "token_kv" else bk.NHDPool.from_block_kv_layers(layers_d)
    t = lambda a: torch.from_numpy(a).to(cuda)
    pool.load_token_major(tm_d, t(load[0]), t(load[1]))
    pool.check()
    assert sha(np.stack([_to_np(x).view(np.uint16).reshape(layers[0].shape) for x in layers_d])) == e["layers_after_load_sha256"]
    pool.store_token_major(tm_d, t(store[0]), t(store[1]))
    pool.check()
    assert sha(_to_np(tm_d)) == e["tm_after_store_sha256"]
