"""Parity of the HIP path against the CPU oracle, through the C ABI, on a real GPU.

Bit-exact is the bar everywhere: this path moves bytes. Every comparison is on raw bytes, so NaN
payloads and fp8 bit patterns count.
"""
import hashlib
import json
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _announce(msg):
    print(f"[case] {msg}", flush=True)


def _rand_pool(rng, n_planes, n_pages, tile_bytes):
    return rng.integers(0, 256, size=(n_planes, n_pages, tile_bytes), dtype=np.uint8)


def _to_np(t):
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()


@pytest.fixture(scope="module")
def bk(lib):
    import bikv_pagecopy
    return bikv_pagecopy


# ---- configuration 1, against the committed digests and the oracle ------------------------------
@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
def test_config1_gather_scatter_bit_exact(bk, oracle, cuda, layout):
    from bikv_pagecopy import workloads
    _announce(f"config1 {layout}")
    with open(os.path.join(GOLDEN, "config1.json")) as f:
        g = json.load(f)
    shape = workloads.SHAPES["tiny"]
    wl = workloads.named("tiny")
    pool_h = np.random.default_rng(0).standard_normal(
        (shape.n_planes, shape.n_pages, shape.tile_bytes // 2)).astype(np.float16)
    pool_d = torch.from_numpy(pool_h).to(cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    batch = pool.make_batch(wl["gather"], layout)
    staging, _ = pool.gather(batch)
    pool.check()
    got = _to_np(staging)
    want = oracle.gather_layered_c(pool_h, wl["gather"], layout)
    assert got.tobytes() == want.tobytes()
    assert hashlib.sha256(got.tobytes()).hexdigest() == g[layout]["staging_sha256"]
    # the per-request view is the contiguous [64, 16, 2, 64] buffer per plane the config asks for
    v = batch.request_view(staging.view(torch.float16), 0)
    if layout == "layer_major":
        assert v.shape == (2, 64, 16 * 2 * 64)
        assert torch.equal(v[1].cpu(), torch.from_numpy(pool_h[1, wl["gather"][0]]))
    sbatch = pool.make_batch(wl["scatter"], layout)
    pool.scatter(sbatch, staging)
    pool.check()
    oracle.scatter_layered_c(pool_h, wl["scatter"], want, layout)
    after = _to_np(pool_d)
    assert after.tobytes() == pool_h.tobytes()
    assert hashlib.sha256(after.tobytes()).hexdigest() == g[layout]["pool_after_scatter_sha256"]


# ---- the other four shapes with scaled-down pools -----------------------------------------------
def _run_shape(bk, oracle, cuda, shape, wl, layout, seed):
    rng = np.random.default_rng(seed)
    pool_h = _rand_pool(rng, shape.n_planes, shape.n_pages, shape.tile_bytes)
    scale_h = _rand_pool(rng, shape.n_planes, shape.n_pages, shape.scale_tile_bytes) if shape.scales else None
    pool_d = torch.from_numpy(pool_h).to(cuda)
    scale_d = torch.from_numpy(scale_h).to(cuda) if shape.scales else None
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1, scale=scale_d)
    batch = pool.make_batch(wl["gather"], layout)
    staging, sstaging = pool.gather(batch)
    pool.check()
    want = oracle.gather_layered_c(pool_h, wl["gather"], layout)
    assert _to_np(staging).tobytes() == want.tobytes()
    if shape.scales:
        swant = oracle.gather_layered_c(scale_h, wl["gather"], layout)
        assert _to_np(sstaging).tobytes() == swant.tobytes()
    if wl.get("scatter"):
        # scatter the first len(scatter) requests' worth of staged data into fresh pages
        sreq = wl["scatter"]
        src_reqs = [rng.permutation(shape.n_pages)[: len(r)] for r in sreq]
        sb_src = pool.make_batch(src_reqs, layout)
        st2, sst2 = pool.gather(sb_src)
        pool.check()
        w2 = oracle.gather_layered_c(pool_h, src_reqs, layout)
        sb = pool.make_batch(sreq, layout)
        pool.scatter(sb, st2, sst2)
        pool.check()
        oracle.scatter_layered_c(pool_h, sreq, w2, layout)
        assert _to_np(pool_d).tobytes() == pool_h.tobytes()
        if shape.scales:
            sw2 = oracle.gather_layered_c(scale_h, src_reqs, layout)
            oracle.scatter_layered_c(scale_h, sreq, sw2, layout)
            assert _to_np(scale_d).tobytes() == scale_h.tobytes()


@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
def test_qwen2_1p5b_shape_scaled_pool(bk, oracle, cuda, layout):
    from bikv_pagecopy import workloads as w
    shape = w.SHAPES["qwen2_1p5b"].scaled(384)   # 8 KiB tiles, 56 planes: 2 tiles per unrolled pass
    wl = w.uniform_requests(shape, 6, 512, 1024, seed=2)
    _announce(f"qwen2_1p5b scaled {layout}: {sum(map(len, wl['gather']))} pages")
    _run_shape(bk, oracle, cuda, shape, wl, layout, 102)


def test_qwen2_7b_shape_scaled_pool_with_duplicates(bk, oracle, cuda):
    from bikv_pagecopy import workloads as w
    shape = w.SHAPES["qwen2_7b"].scaled(256)     # 16 KiB tiles
    wl = w.mixed_gather_scatter(shape, 6, 256, 1024, seed=3, dup_fraction=0.10)
    g = np.concatenate(wl["gather"])
    assert len(set(g.tolist())) < len(g), "workload must contain duplicate gather ids"
    _announce(f"qwen2_7b scaled: {len(g)} gather pages, dup present")
    _run_shape(bk, oracle, cuda, shape, wl, "layer_major", 103)


def test_llama3_8b_shape_scaled_pool(bk, oracle, cuda):
    from bikv_pagecopy import workloads as w
    shape = w.SHAPES["llama3_8b"].scaled(48)      # 64 KiB tiles: four unrolled passes per tile
    wl = w.lognormal_requests(shape, 5, 256, 1024, seed=4)
    _announce(f"llama3_8b scaled: {sum(map(len, wl['gather']))} pages")
    _run_shape(bk, oracle, cuda, shape, wl, "layer_major", 104)


@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
def test_llama3_70b_fp8_payload_and_scales_move_together(bk, oracle, cuda, layout):
    from bikv_pagecopy import workloads as w
    shape = w.SHAPES["llama3_70b_fp8"].scaled(96)  # 16 KiB payload + 32 B scales, 160 planes
    wl = w.zipf_requests(shape, 12, 16, 512, seed=5)
    assert wl["scatter"], "need a scatter leg"
    _announce(f"llama3_70b_fp8 scaled {layout}: {sum(map(len, wl['gather']))} pages")
    _run_shape(bk, oracle, cuda, shape, wl, layout, 105)


# ---- shapes the fast mover does not take ----------------------------------------------------------
@pytest.mark.parametrize("tile_bytes", [16, 48, 100, 1000, 4096 * 3, 4096 + 16, 2, 7])
def test_odd_tile_sizes(bk, oracle, cuda, tile_bytes):
    _announce(f"odd tile {tile_bytes}")
    rng = np.random.default_rng(tile_bytes)
    pool_h = _rand_pool(rng, 3, 70, tile_bytes)
    pool_d = torch.from_numpy(pool_h).to(cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    reqs = [rng.permutation(70)[:33], np.array([4, 4, 4]), rng.permutation(70)[:1]]
    batch = pool.make_batch(reqs)
    staging, _ = pool.gather(batch)
    pool.check()
    assert _to_np(staging).tobytes() == oracle.gather_layered_c(pool_h, reqs).tobytes()


@pytest.mark.parametrize("tile_bytes", [24576, 40960, 1536, 528, 1008, 4096 + 16, 3 * 1024, 7 * 1024 + 512])
@pytest.mark.parametrize("order", [0, 1])
def test_wave_mover_with_piece_counts_that_are_not_powers_of_two(bk, oracle, cuda, tile_bytes, order):
    """6 KV heads give 24 KiB tiles (24 pieces of 1 KiB); other sizes end in a ragged piece."""
    _announce(f"wave mover tile {tile_bytes} order {order}")
    rng = np.random.default_rng(tile_bytes + order)
    pool_h = _rand_pool(rng, 5, 40, tile_bytes)
    pool_d = torch.from_numpy(pool_h).to(cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    reqs = [rng.permutation(40)[:13], np.array([7, 7]), rng.permutation(40)[:1]]
    try:
        bk.set_tuning(order=order, log2_chunk=2 if order else -1)
        for layout in ("layer_major", "page_major"):
            batch = pool.make_batch(reqs, layout)
            st = torch.full((batch.n_slots * tile_bytes + 32,), 0xA5, dtype=torch.uint8, device=cuda)
            pool.gather(batch, st[: batch.n_slots * tile_bytes])
            pool.check()
            assert _to_np(st[: batch.n_slots * tile_bytes]).tobytes() == oracle.gather_layered_c(pool_h, reqs, layout).tobytes()
            assert torch.all(st[batch.n_slots * tile_bytes:] == 0xA5)      # nothing past the last ragged piece
        perm = rng.permutation(40)
        sreqs = [perm[:9], perm[9:12]]
        sb = pool.make_batch(sreqs)
        src = torch.from_numpy(rng.integers(0, 256, size=sb.n_slots * tile_bytes, dtype=np.uint8)).to(cuda)
        pool.scatter(sb, src)
        pool.check()
        oracle.scatter_layered_c(pool_h, sreqs, src.cpu().numpy())
        assert _to_np(pool_d).tobytes() == pool_h.tobytes()
    finally:
        bk.set_tuning(order=-1, log2_chunk=-1)


def test_misaligned_pool_and_staging(bk, oracle, cuda):
    """Pool planes and staging that start 2 bytes off a 16-byte boundary take the narrow mover."""
    _announce("misaligned")
    rng = np.random.default_rng(77)
    n_planes, n_pages, tile = 2, 40, 8192
    backing = torch.zeros(n_planes * n_pages * tile + 64, dtype=torch.uint8, device=cuda)
    pool_h = _rand_pool(rng, n_planes, n_pages, tile)
    view = backing[2: 2 + pool_h.size].view(n_planes, n_pages, tile)
    view.copy_(torch.from_numpy(pool_h))
    assert view.data_ptr() % 16 == 2
    pool = bk.PagedKVPool([view[q].data_ptr() for q in range(n_planes)], n_pages, tile, tile, cuda)
    reqs = [rng.permutation(n_pages)[:17]]
    batch = pool.make_batch(reqs)
    st_back = torch.zeros(batch.n_slots * tile + 64, dtype=torch.uint8, device=cuda)
    staging = st_back[6: 6 + batch.n_slots * tile]
    pool.gather(batch, staging)
    pool.check()
    assert _to_np(staging).tobytes() == oracle.gather_layered_c(pool_h, reqs).tobytes()
    assert not st_back[:6].any() and not st_back[6 + batch.n_slots * tile:].any()


def test_kv_adjacent_layer_layout(bk, oracle, cuda):
    """Per-layer [pages, 2, block, heads, dim] tensors as in Model/qwen2.py:532-536."""
    _announce("kv-adjacent layers")
    rng = np.random.default_rng(31)
    L, N, P, H, D = 3, 24, 16, 2, 128
    layers_h = [rng.standard_normal((N, 2, P, H, D)).astype(np.float16) for _ in range(L)]
    layers_d = [torch.from_numpy(a).to(cuda) for a in layers_h]
    pool = bk.PagedKVPool.from_layers_kv_adjacent(layers_d)
    assert pool.n_planes == 2 * L and pool.page_stride_bytes == 2 * pool.tile_bytes
    # the oracle's plane-major view of the same data
    planes_h = np.stack([layers_h[l][:, k].reshape(N, -1) for l in range(L) for k in range(2)])
    reqs = [rng.permutation(N)[:9], rng.permutation(N)[:4]]
    batch = pool.make_batch(reqs)
    staging, _ = pool.gather(batch)
    pool.check()
    want = oracle.gather_layered_c(np.ascontiguousarray(planes_h), reqs)
    assert _to_np(staging).tobytes() == want.view(np.uint8).tobytes()
    # scatter back into other pages and compare each layer tensor
    perm = rng.permutation(N)
    sreqs = [perm[:9], perm[9:13]]
    pool.scatter(pool.make_batch(sreqs), staging)
    pool.check()
    planes_c = np.ascontiguousarray(planes_h)
    oracle.scatter_layered_c(planes_c, sreqs, want)
    for l in range(L):
        got = layers_d[l].cpu().numpy()
        for k in range(2):
            assert got[:, k].reshape(N, -1).tobytes() == planes_c[2 * l + k].tobytes()


# ---- edge cases ----------------------------------------------------------------------------------
@pytest.mark.parametrize("P,H,D,dtype", [
    (16, 2, 128, torch.float16),      # the Worker's own shape: 512-byte rows, 8 KiB tiles
    (16, 4, 128, torch.bfloat16),     # 1 KiB rows: one piece of the wave mover per row
    (16, 8, 128, torch.float16),      # 2 KiB rows
    (8, 3, 64, torch.float16),        # 384-byte rows (not a power of two)
    (4, 1, 8, torch.float32),         # 32-byte rows, 128-byte tiles: the segment mover
    (5, 2, 24, torch.uint8),          # 48-byte rows, 240-byte tiles
])
@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
def test_worker_token_interleaved_layers(bk, oracle, cuda, P, H, D, dtype, layout):
    """The Worker's per-layer cache [blocks*block, 2, heads, dim] (Worker/Worker.py:74-78) as the pool:
    a (page, K|V) tile is `block` rows of heads*dim elements, two rows apart."""
    _announce(f"worker-form pool P={P} H={H} D={D} {dtype} {layout}")
    rng = np.random.default_rng(P * 1000 + H * 10 + D)
    es = torch.empty((), dtype=dtype).element_size()
    np_dt = {1: np.uint8, 2: np.uint16, 4: np.uint32}[es]
    L, blocks = 3, 37
    layers_h = [rng.integers(0, 256, size=(blocks * P, 2, H, D, es), dtype=np.uint8).view(np_dt)[..., 0].copy() for _ in range(L)]
    layers_d = [torch.from_numpy(a.view(np.uint8)).to(cuda).view(dtype).view(a.shape) for a in layers_h]
    pool = bk.PagedKVPool.from_token_kv_layers(layers_d, P)
    assert pool.n_planes == 2 * L and pool.tile_bytes == P * H * D * es
    planes_h = oracle.planes_of_token_kv_layers(layers_h, P).view(np.uint8)
    reqs = [rng.permutation(blocks)[:15], np.array([3, 3]), rng.permutation(blocks)[:1], np.array([], dtype=np.int64)]
    batch = pool.make_batch(reqs, layout)
    st, _ = pool.gather(batch)
    pool.check()
    assert _to_np(st).tobytes() == oracle.gather_layered_c(planes_h, reqs, layout).tobytes()
    perm = rng.permutation(blocks)
    sreqs = [perm[:9], perm[9:20]]
    sb = pool.make_batch(sreqs, layout)
    src = rng.integers(0, 256, size=sb.n_slots * pool.tile_bytes, dtype=np.uint8)
    pool.scatter(sb, torch.from_numpy(src).to(cuda))
    pool.check()
    oracle.scatter_layered_c(planes_h, sreqs, src, layout)
    want = oracle.token_kv_layers_of_planes(planes_h.view(np_dt), P, H, D)
    for l in range(L):
        assert _to_np(layers_d[l]).tobytes() == want[l].tobytes(), f"layer {l}"
    # a window of planes that starts on a V plane
    d = batch.desc(plane_begin=1, plane_count=3)
    win = torch.full((batch.n_slots * pool.tile_bytes,), 0xA5, dtype=torch.uint8, device=cuda)
    from bikv_pagecopy import _lib
    import ctypes as C
    _lib.check(_lib.load().bikv_gather_pages(pool._h, C.byref(d), win.data_ptr(), win.numel(), None, 0,
                                             C.c_void_p(torch.cuda.current_stream(cuda).cuda_stream)))
    pool.check()
    full = oracle.gather_layered_c(planes_h, reqs, layout).reshape(batch.n_slots, pool.tile_bytes)
    got = _to_np(win).reshape(batch.n_slots, pool.tile_bytes)
    n_pl = pool.n_planes
    for r in range(len(reqs)):
        m = len(reqs[r])
        if m == 0:
            continue
        s0 = int(batch.req_first_slot[r])
        blk_got, blk_want = got[s0:s0 + m * n_pl], full[s0:s0 + m * n_pl]
        view = (lambda a: a.reshape(n_pl, m, -1)) if layout == "layer_major" else (lambda a: a.reshape(m, n_pl, -1).transpose(1, 0, 2))
        g3, w3 = view(blk_got), view(blk_want)
        assert np.array_equal(g3[1:4], w3[1:4]) and (g3[0] == 0xA5).all() and (g3[4:] == 0xA5).all()
    pool.close()


@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
def test_half_kib_rows_of_the_worker_shape_match_the_oracle_in_every_walk(bk, oracle, cuda, layout):
    """The Worker's own shape (2 KV heads x 128 x fp16: 512-byte rows, K and V of a token adjacent, so that a
    wave's KiB of a tile is two half-KiB pieces of the pool): every walk of the wave mover against the oracle,
    and a rejected page id."""
    _announce(f"half-KiB rows {layout}")
    rng = np.random.default_rng(311)
    P, H, D, L, blocks = 16, 2, 128, 5, 70
    layers_h = [rng.integers(0, 65536, size=(blocks * P, 2, H, D), dtype=np.uint16) for _ in range(L)]
    planes_h = oracle.planes_of_token_kv_layers(layers_h, P).view(np.uint8)
    reqs = [rng.permutation(blocks)[:33], np.array([5, 5, 9]), rng.permutation(blocks)[:1]]
    want = oracle.gather_layered_c(planes_h, reqs, layout).tobytes()
    perm = rng.permutation(blocks)
    sreqs = [perm[:21], perm[21:40]]
    for order, lc in ((-1, -1), (0, 0), (1, 0), (1, 2), (1, 5)):
        bk.set_tuning(order=order, log2_chunk=lc)
        layers_d = [torch.from_numpy(a.view(np.int16)).to(cuda).view(torch.float16) for a in layers_h]
        pool = bk.PagedKVPool.from_token_kv_layers(layers_d, P)
        batch = pool.make_batch(reqs, layout)
        st, _ = pool.gather(batch)
        pool.check()
        assert _to_np(st).tobytes() == want, (order, lc)
        sb = pool.make_batch(sreqs, layout, check_unique=True)
        src = rng.integers(0, 256, size=sb.n_slots * pool.tile_bytes, dtype=np.uint8)
        pool.scatter(sb, torch.from_numpy(src).to(cuda))
        pool.check()
        ph = planes_h.copy()
        oracle.scatter_layered_c(ph, sreqs, src, layout)
        back = oracle.token_kv_layers_of_planes(ph.view(np.uint16), P, H, D)
        for l in range(L):
            assert _to_np(layers_d[l]).tobytes() == back[l].tobytes(), (order, lc, l)
        # a page id outside the pool: that page is skipped and reported, its neighbours still move
        bad = pool.make_batch([[2, blocks + 3, 7]], layout)
        st2 = torch.full((bad.n_slots * pool.tile_bytes,), 0xA5, dtype=torch.uint8, device=cuda)
        pool.gather(bad, st2)
        with pytest.raises(RuntimeError, match="page-id"):
            pool.check()
        v = bad.request_view(st2, 0)
        good = oracle.gather_layered_c(ph, [np.array([2, 7])], layout)
        gv = good.reshape(2 * L, 2, -1) if layout == "layer_major" else good.reshape(2, 2 * L, -1)
        if layout == "layer_major":
            assert np.array_equal(_to_np(v[:, 0]), gv[:, 0]) and np.array_equal(_to_np(v[:, 2]), gv[:, 1])
            assert bool((v[:, 1] == 0xA5).all())
        else:
            assert np.array_equal(_to_np(v[0]), gv[0]) and np.array_equal(_to_np(v[2]), gv[1])
            assert bool((v[1] == 0xA5).all())
        pool.close()


def test_empty_batch_and_empty_requests(bk, oracle, cuda):
    _announce("empty")
    pool_d = torch.zeros((2, 8, 4096), dtype=torch.uint8, device=cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    b = pool.make_batch([])
    st, _ = pool.gather(b)
    pool.check()
    assert st.numel() == 0
    b = pool.make_batch([[], [], []])
    st, _ = pool.gather(b)
    pool.check()
    assert st.numel() == 0


def test_nan_payloads_and_all_bit_patterns_survive(bk, cuda):
    _announce("bit patterns")
    allbits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.float16)  # every fp16 pattern
    pool_d = allbits.repeat(2 * 16).view(2, 16, 65536).contiguous().to(cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    b = pool.make_batch([[15, 0, 15]])
    st, _ = pool.gather(b)
    pool.check()
    got = st.view(torch.int16).view(2, 3, 65536).cpu()
    assert torch.equal(got[0, 0], allbits.view(torch.int16)) and torch.equal(got[1, 2], allbits.view(torch.int16))


def test_plane_subrange_and_slot_bias(bk, oracle, cuda, lib):
    """The windowed form the host pipeline uses: planes [q0, q0+k) into a window of the image."""
    import ctypes as C
    from bikv_pagecopy import _lib
    _announce("plane window")
    rng = np.random.default_rng(55)
    pool_h = _rand_pool(rng, 8, 30, 4096)
    pool_d = torch.from_numpy(pool_h).to(cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    reqs = [rng.permutation(30)[:11]]
    batch = pool.make_batch(reqs)
    want = oracle.gather_layered_c(pool_h, reqs).reshape(8, 11, 4096)
    window = torch.full((3 * 11 * 4096,), 0xA5, dtype=torch.uint8, device=cuda)
    d = batch.desc(plane_begin=2, plane_count=3, slot_bias=2 * 11)
    _lib.check(lib.bikv_gather_pages(pool._h, C.byref(d), window.data_ptr(), window.numel(), None, 0,
                                     C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    pool.check()
    assert _to_np(window).tobytes() == want[2:5].tobytes()


def test_out_of_range_ids_and_slots_are_skipped_and_reported(bk, oracle, cuda):
    """A bad page id or a staging buffer that is too small must not touch memory outside the
    buffers: the tile is skipped, the call reports it, every other tile is still moved."""
    _announce("bounds rejection")
    rng = np.random.default_rng(66)
    pool_h = _rand_pool(rng, 2, 20, 4096)
    pool_d = torch.from_numpy(pool_h).to(cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    reqs = [np.array([3, 20, 5, -1, 7], dtype=np.int64)]
    batch = pool.make_batch(reqs)
    st = torch.full((batch.n_slots * 4096,), 0xA5, dtype=torch.uint8, device=cuda)
    pool.gather(batch, st)
    with pytest.raises(RuntimeError, match="page-id"):
        pool.check()
    got = _to_np(st).reshape(2, 5, 4096)
    for j, pid in enumerate(reqs[0]):
        if 0 <= pid < 20:
            assert np.array_equal(got[:, j], pool_h[:, pid])
        else:
            assert np.all(got[:, j] == 0xA5)
    pool.check()  # status was cleared by the failing check
    good = pool.make_batch([np.array([1, 2, 3, 4])])
    small = torch.full((2 * 4 * 4096 - 4096,), 0xA5, dtype=torch.uint8, device=cuda)  # one slot short
    pool.gather(good, small)
    with pytest.raises(RuntimeError, match="destination-range"):
        pool.check()
    # scatter with a bad id leaves the pool untouched for that id
    before = _to_np(pool_d).copy()
    bad = pool.make_batch([np.array([25])])
    pool.scatter(bad, torch.zeros(2 * 4096, dtype=torch.uint8, device=cuda))
    with pytest.raises(RuntimeError, match="page-id"):
        pool.check()
    assert _to_np(pool_d).tobytes() == before.tobytes()


def test_tuning_knobs_do_not_change_results(bk, oracle, cuda):
    _announce("launch geometry independence")
    rng = np.random.default_rng(88)
    pool_h = _rand_pool(rng, 4, 64, 16384)
    pool_d = torch.from_numpy(pool_h).to(cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    reqs = [rng.permutation(64)[:37], rng.permutation(64)[:5]]
    want = oracle.gather_layered_c(pool_h, reqs).tobytes()
    batch = pool.make_batch(reqs)
    sreqs = [rng.permutation(64)[:42]]
    sbatch = pool.make_batch(sreqs)
    src = torch.from_numpy(rng.integers(0, 256, size=sbatch.n_slots * 16384, dtype=np.uint8)).to(cuda)
    want_pool = pool_h.copy()
    oracle.scatter_layered_c(want_pool, sreqs, src.cpu().numpy())
    try:
        # seg 0 = wave mover (wave_block lanes per workgroup); seg > 0 = LDS-staged segment mover
        cases = [dict(seg=0, wave_block=wb, nontemporal=nt) for wb in (64, 128, 256) for nt in (-1, 0, 1, 4)]
        # wave mover walks: plane by plane, or chunks of 2^k pages with their planes together
        cases += [dict(seg=0, wave_block=64, order=o, log2_chunk=lc) for o in (0, 1) for lc in (-1, 0, 1, 3, 6, 10)]
        cases += [dict(seg=seg, unroll=u, nontemporal=nt) for seg in (1, 3, 16, 256) for u in (1, 2, 4, 8)
                  for nt in (0, 1)]
        for kw in cases:
            bk.set_tuning(**kw)
            st = torch.zeros(batch.n_slots * 16384, dtype=torch.uint8, device=cuda)
            pool.gather(batch, st)
            pool.check()
            assert _to_np(st).tobytes() == want, kw
            pool_d.copy_(torch.from_numpy(pool_h))
            pool.scatter(sbatch, src)
            pool.check()
            assert _to_np(pool_d).tobytes() == want_pool.tobytes(), kw
            pool_d.copy_(torch.from_numpy(pool_h))
    finally:
        bk.set_tuning(seg=0, wave_block=64, unroll=4, nontemporal=-1, order=-1, log2_chunk=-1)


# ---- run copy (reference API) -------------------------------------------------------------------
@pytest.mark.parametrize("dtype,run_elems", [
    (torch.float16, 14336 * 16), (torch.bfloat16, 4096), (torch.float32, 1000), (torch.float64, 33),
    (torch.uint8, 5), (torch.uint8, 2049), (torch.float16, 8), (torch.float16, 1029),
    (torch.float16, 512), (torch.uint8, 1023), (torch.uint8, 16384)])
@pytest.mark.parametrize("run_group", [1, 0])
def test_copy_runs_gather_and_scatter(bk, oracle, cuda, dtype, run_elems, run_group):
    _announce(f"copy_runs {dtype} run_elems={run_elems} run_group={run_group}")
    bk.set_tuning(run_group=run_group)
    rng = np.random.default_rng(run_elems)
    es = torch.empty((), dtype=dtype).element_size()
    n_pages, n = 37, 19
    src_h = rng.integers(0, 256, size=n_pages * run_elems * es, dtype=np.uint8)
    src_d = torch.from_numpy(src_h).to(cuda).view(dtype)
    ids = rng.integers(0, n_pages, size=n)                  # duplicates allowed on the source side
    so = ids * run_elems
    do = rng.permutation(n).astype(np.int64) * run_elems    # dense but out of order
    dst_d = torch.full((n * run_elems * es,), 0xA5, dtype=torch.uint8, device=cuda).view(dtype)
    bk.copy_runs(src_d, dst_d, torch.from_numpy(so).to(cuda), torch.from_numpy(do).to(cuda), run_elems)
    from bikv_pagecopy import runs
    runs.check(cuda)
    dst_h = np.full(n * run_elems * es, 0xA5, dtype=np.uint8)
    np_dt = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[es]
    assert oracle.copy_runs_c(src_h.view(np_dt), dst_h.view(np_dt), so, do, run_elems) == 0
    assert _to_np(dst_d).tobytes() == dst_h.tobytes()
    # scatter back: dense source, scattered unique destinations
    back_ids = rng.permutation(n_pages)[:n].astype(np.int64) * run_elems
    pool2_d = torch.zeros_like(src_d)
    bk.copy_runs(dst_d, pool2_d, torch.from_numpy(do).to(cuda), torch.from_numpy(back_ids).to(cuda), run_elems)
    runs.check(cuda)
    pool2_h = np.zeros_like(src_h)
    oracle.copy_runs_c(dst_h.view(np_dt), pool2_h.view(np_dt), do, back_ids, run_elems)
    assert _to_np(pool2_d).tobytes() == pool2_h.tobytes()
    bk.set_tuning(run_group=1)


def test_copy_runs_element_offsets_that_break_16_byte_alignment(bk, oracle, cuda):
    """fp16 element offsets need only be 2-byte aligned: every run picks its own access width."""
    _announce("copy_runs unaligned offsets")
    rng = np.random.default_rng(12)
    run = 3000
    src_h = rng.integers(0, 65536, size=40000, dtype=np.uint16)
    so = np.array([0, 1, 2, 3, 4, 8, 1001, 20000], dtype=np.int64)
    do = np.array([0, 3001, 6003, 9008, 12012, 15015, 18023, 21024], dtype=np.int64)
    dst_h = np.full(25000, 0xA5A5, dtype=np.uint16)
    oracle.copy_runs_c(src_h, dst_h, so, do, run)
    src_d = torch.from_numpy(src_h.view(np.int16)).to(cuda).view(torch.float16)
    dst_d = torch.from_numpy(np.full(25000, 0xA5A5, dtype=np.uint16).view(np.int16)).to(cuda).view(torch.float16)
    bk.copy_runs(src_d, dst_d, torch.from_numpy(so).to(cuda), torch.from_numpy(do).to(cuda), run)
    from bikv_pagecopy import runs
    runs.check(cuda)
    assert _to_np(dst_d).tobytes() == dst_h.tobytes()


@pytest.mark.parametrize("pinned_source", [False, True])
def test_copy_runs_ragged_lengths(bk, oracle, cuda, pinned_source):
    """Every run has its own length: zero, one element, around 16-byte and 1-KiB piece boundaries,
    the maximum; offsets only element-aligned."""
    _announce(f"copy_runs ragged, pinned source={pinned_source}")
    from bikv_pagecopy import runs
    rng = np.random.default_rng(61)
    max_run = 5000
    fixed = [0, 1, 7, 8, 9, 511, 512, 513, 1024, 4095, 4096, max_run]
    lens = np.array(fixed + rng.integers(0, max_run + 1, size=40).tolist(), dtype=np.int64)
    n = len(lens)
    src_h = rng.integers(0, 65536, size=60000, dtype=np.uint16)
    so = rng.integers(0, 60000 - max_run, size=n).astype(np.int64)
    do = np.concatenate([[0], np.cumsum(lens + rng.integers(0, 3, size=n))[:-1]]).astype(np.int64)
    total = int(do[-1] + lens[-1]) + 5
    dst_h = np.full(total, 0xA5A5, dtype=np.uint16)
    assert oracle.copy_runs_ragged_c(src_h, dst_h, so, do, lens, max_run) == 0
    src_t = torch.from_numpy(src_h.view(np.int16)).view(torch.float16)
    src_t = src_t.pin_memory() if pinned_source else src_t.to(cuda)
    dst_d = torch.from_numpy(np.full(total, 0xA5A5, dtype=np.uint16).view(np.int16)).to(cuda).view(torch.float16)
    bk.copy_runs(src_t, dst_d, torch.from_numpy(so).to(cuda), torch.from_numpy(do).to(cuda), max_run,
                 device=cuda, run_lens=torch.from_numpy(lens).to(cuda))
    runs.check(cuda)
    assert _to_np(dst_d).tobytes() == dst_h.tobytes()
    # token units: offsets and lengths count blocks of 24 elements
    unit, max_units = 24, 16
    lens_u = rng.integers(0, max_units + 1, size=30).astype(np.int64)
    so_u = rng.integers(0, 60000 // unit - max_units, size=30).astype(np.int64)
    do_u = np.concatenate([[0], np.cumsum(lens_u)[:-1]]).astype(np.int64)
    want = np.full(int(lens_u.sum()) * unit, 0xA5A5, dtype=np.uint16)
    assert oracle.copy_runs_ragged_c(src_h, want, so_u, do_u, lens_u, max_units, unit_elems=unit) == 0
    got = torch.from_numpy(np.full(want.size, 0xA5A5, dtype=np.uint16).view(np.int16)).to(cuda).view(torch.float16)
    bk.copy_runs(src_t, got, torch.from_numpy(so_u).to(cuda), torch.from_numpy(do_u).to(cuda), max_units * unit,
                 device=cuda, run_lens=torch.from_numpy(lens_u).to(cuda), unit_elems=unit)
    runs.check(cuda)
    assert _to_np(got).tobytes() == want.tobytes()


def test_copy_runs_ragged_reports_bad_lengths(bk, cuda):
    _announce("copy_runs ragged bounds")
    from bikv_pagecopy import runs
    src = torch.arange(0, 4096, dtype=torch.int16, device=cuda)
    dst = torch.zeros(4096, dtype=torch.int16, device=cuda)
    so = torch.tensor([0, 100, 200, 4090], dtype=torch.int64, device=cuda)
    do = torch.tensor([0, 100, 200, 300], dtype=torch.int64, device=cuda)
    lens = torch.tensor([50, -3, 65, 10], dtype=torch.int64, device=cuda)     # ok, negative, above max, src overrun
    bk.copy_runs(src, dst, so, do, 64, run_lens=lens)
    with pytest.raises(RuntimeError, match="source-range"):
        runs.check(cuda)
    assert torch.equal(dst[:50], src[:50]) and not dst[50:].any()
    with pytest.raises(RuntimeError, match="differ in length"):
        bk.copy_runs(src, dst, so, do, 64, run_lens=lens[:2].contiguous())


def test_copy_runs_rejects_offsets_outside_the_buffers(bk, cuda):
    _announce("copy_runs bounds")
    from bikv_pagecopy import runs
    src = torch.arange(0, 4096, dtype=torch.int16, device=cuda)
    dst = torch.zeros(4096, dtype=torch.int16, device=cuda)
    so = torch.tensor([0, 4000, -5, 1024], dtype=torch.int64, device=cuda)
    do = torch.tensor([0, 1024, 2048, 3500], dtype=torch.int64, device=cuda)
    bk.copy_runs(src, dst, so, do, 1024)
    with pytest.raises(RuntimeError, match="source-range"):
        runs.check(cuda)
    assert torch.equal(dst[:1024], src[:1024]) and not dst[1024:].any()
    with pytest.raises(RuntimeError, match="contiguous"):
        bk.copy_runs(src[::2], dst, so, do, 4)
    with pytest.raises(RuntimeError, match="CUDA"):
        bk.copy_runs(src, dst, so.cpu(), do, 4)


def test_copy_runs_zero_copy_from_pinned_host(bk, oracle, cuda):
    """The zero_copy_page_kernel form: the source is pinned host memory read by the GPU."""
    _announce("copy_runs pinned source")
    rng = np.random.default_rng(13)
    run = 14336 * 4
    src_h = rng.integers(0, 65536, size=12 * run, dtype=np.uint16)
    pinned = torch.from_numpy(src_h.view(np.int16)).pin_memory().view(torch.float16)
    ids = rng.permutation(12)[:7].astype(np.int64)
    so, do = ids * run, np.arange(7, dtype=np.int64) * run
    dst = torch.zeros(7 * run, dtype=torch.float16, device=cuda)
    bk.copy_runs(pinned, dst, torch.from_numpy(so).to(cuda), torch.from_numpy(do).to(cuda), run, device=cuda)
    from bikv_pagecopy import runs
    runs.check(cuda)
    want = np.zeros(7 * run, dtype=np.uint16)
    oracle.copy_runs_c(src_h, want, so, do, run)
    assert _to_np(dst).tobytes() == want.tobytes()


# ---- seeded random sweep ------------------------------------------------------------------------
def test_random_pools_batches_and_knobs_match_oracle(bk, oracle, cuda):
    """Forty seeded cases over everything a caller can vary at once: plane count, pool size, tile size
    (wave-mover shapes, ragged pieces, tiny and odd tiles), a page stride wider than the tile, an
    optional scale class, staging layout, duplicate and out-of-order ids, empty requests, walk order and
    chunk, workgroup size. Gather against the oracle, then scatter into other pages; the gaps between
    tiles must keep their canary."""
    rng = np.random.default_rng(2024)
    tiles = [16, 80, 1000, 1024, 3072, 4096, 5000, 8192, 16384, 20480, 65536]
    try:
        for case in range(40):
            n_planes = int(rng.integers(1, 9))
            n_pages = int(rng.integers(6, 50))
            tile = int(rng.choice(tiles))
            gap = int(rng.choice([0, 0, 16, 64, 4096])) if tile % 16 == 0 else 0
            stile = int(rng.choice([0, 0, 4, 32, 48]))
            layout = str(rng.choice(["layer_major", "page_major"]))
            knobs = dict(order=int(rng.integers(-1, 2)), log2_chunk=int(rng.integers(-1, 5)),
                         wave_block=int(rng.choice([64, 128, 256])), nontemporal=int(rng.choice([-1, 0, 1, 4])))
            _announce(f"random case {case}: planes={n_planes} pages={n_pages} tile={tile}+{gap} scale={stile} {layout} {knobs}")
            bk.set_tuning(**knobs)
            back_h = rng.integers(0, 256, size=(n_planes, n_pages, tile + gap), dtype=np.uint8)
            back_d = torch.from_numpy(back_h).to(cuda)
            pool_h = np.ascontiguousarray(back_h[:, :, :tile])
            sc_h = rng.integers(0, 256, size=(n_planes, n_pages, max(stile, 1)), dtype=np.uint8)
            sc_d = torch.from_numpy(sc_h).to(cuda)
            pool = bk.PagedKVPool([back_d[q].data_ptr() for q in range(n_planes)], n_pages, tile, tile + gap, cuda,
                                  scale_plane_ptrs=[sc_d[q].data_ptr() for q in range(n_planes)] if stile else None,
                                  scale_tile_bytes=stile, scale_page_stride_bytes=stile, keepalive=(back_d, sc_d))
            n_req = int(rng.integers(1, 5))
            g_reqs = [rng.integers(0, n_pages, size=int(rng.integers(0, n_pages))) for _ in range(n_req)]   # duplicates
            gb = pool.make_batch(g_reqs, layout)
            st, sc = pool.gather(gb)
            pool.check()
            assert _to_np(st).tobytes() == oracle.gather_layered_c(pool_h, g_reqs, layout).tobytes(), case
            if stile:
                assert _to_np(sc).tobytes() == oracle.gather_layered_c(sc_h, g_reqs, layout).tobytes(), case
            perm = rng.permutation(n_pages)
            cuts = np.sort(rng.integers(0, n_pages, size=n_req - 1))
            s_reqs = [np.ascontiguousarray(a) for a in np.split(perm[: int(rng.integers(1, n_pages + 1))], [c for c in cuts if c < n_pages])]
            s_reqs = [r for r in s_reqs]
            sb = pool.make_batch(s_reqs, layout)
            src = rng.integers(0, 256, size=sb.n_slots * tile, dtype=np.uint8)
            ssrc = rng.integers(0, 256, size=sb.n_slots * max(stile, 1), dtype=np.uint8)
            pool.scatter(sb, torch.from_numpy(src).to(cuda), torch.from_numpy(ssrc).to(cuda) if stile else None)
            pool.check()
            oracle.scatter_layered_c(pool_h, s_reqs, src, layout)
            got = _to_np(back_d).reshape(n_planes, n_pages, tile + gap)
            assert got[:, :, :tile].tobytes() == pool_h.tobytes(), case
            assert got[:, :, tile:].tobytes() == back_h[:, :, tile:].tobytes(), case      # gaps untouched
            if stile:
                oracle.scatter_layered_c(sc_h, s_reqs, ssrc[: sb.n_slots * stile], layout)
                assert _to_np(sc_d).tobytes() == sc_h.tobytes(), case
            pool.close()
    finally:
        bk.set_tuning(seg=0, wave_block=64, unroll=4, nontemporal=-1, order=-1, log2_chunk=-1)


# ---- HIP graph capture --------------------------------------------------------------------------
def test_gather_scatter_and_run_copy_replay_from_a_hip_graph(bk, oracle, cuda):
    """The asynchronous entry points only launch kernels (no allocation, no memset, no synchronisation),
    so a serving loop can capture them once and replay: every replay is checked against the oracle with
    different pool contents, with eager work and synchronisations between the replays."""
    _announce("graph capture: gather + scatter + copy_runs")
    from bikv_pagecopy import runs
    rng = np.random.default_rng(71)
    n_planes, n_pages, tile = 6, 64, 8192
    pool_h = rng.integers(0, 256, size=(n_planes, n_pages, tile), dtype=np.uint8)
    pool_d = torch.from_numpy(pool_h).to(cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    perm = rng.permutation(n_pages)
    g_reqs = [perm[:9], perm[5:20]]                       # overlapping requests: duplicate reads
    s_reqs = [perm[30:39], perm[40:55]]                   # unique, disjoint from the gathered pages
    gb, sb = pool.make_batch(g_reqs, "layer_major"), pool.make_batch(s_reqs, "layer_major")
    st, _ = pool.empty_staging(gb)
    run = tile // 2
    so = torch.from_numpy(np.arange(0, 4 * run, run, dtype=np.int64)).to(cuda)
    do = torch.from_numpy(np.array([3, 1, 0, 2], dtype=np.int64) * run).to(cuda)
    copy_out = torch.zeros(4 * run, dtype=torch.float16, device=cuda)
    # one eager pass first: per-device set-up (the status block) happens outside the capture
    pool.gather(gb, st)
    pool.check()
    stream = torch.cuda.Stream(device=cuda)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            pool.gather(gb, st)
            pool.scatter(sb, st)
            bk.copy_runs(st.view(torch.float16), copy_out, so, do, run)
    for rep in range(3):
        pool_h = rng.integers(0, 256, size=(n_planes, n_pages, tile), dtype=np.uint8)
        pool_d.copy_(torch.from_numpy(pool_h))            # eager work between replays
        st.fill_(0xA5)
        copy_out.zero_()
        torch.cuda.synchronize(cuda)
        graph.replay()
        torch.cuda.synchronize(cuda)
        pool.check()
        staged = oracle.gather_layered_c(pool_h, g_reqs, "layer_major")
        want_pool = pool_h.copy()
        oracle.scatter_layered_c(want_pool, s_reqs, staged, "layer_major")
        assert _to_np(st).tobytes() == staged.tobytes(), rep
        assert _to_np(pool_d).tobytes() == want_pool.tobytes(), rep
        want_copy = np.zeros(4 * run, dtype=np.uint16)
        oracle.copy_runs_c(staged.view(np.uint16).reshape(-1), want_copy, so.cpu().numpy(), do.cpu().numpy(), run)
        assert _to_np(copy_out).tobytes() == want_copy.tobytes(), rep
    runs.check(cuda)
    pool.close()


def test_plain_c_program_drives_the_library(bk, cuda):
    """tests/c_client/abi_client.c: gcc-built, includes only include/bikv_pagecopy.h, links only the
    shared library. Run copy, ragged run copy, layered gather/scatter and a rejected page id."""
    import os
    import subprocess
    _announce("plain-C client of the ABI")
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_client")
    exe = os.path.join(here, "abi_client")
    if not os.path.exists(exe):                    # loads what is built; builds only when nothing is
        subprocess.run(["make", "-C", here], check=True, capture_output=True, timeout=100)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0 and "abi_client: ok" in r.stdout, (r.returncode, r.stdout, r.stderr)


def test_duplicate_scatter_destinations_are_refused_in_debug_mode(bk, cuda):
    """With the debug check on (BIKV_DEBUG_UNIQUE=1 or the tuning knob), a scatter whose page ids repeat
    is refused before it launches; a gather with the same ids is legal."""
    print("[case] duplicate destinations, debug check", flush=True)
    pool_d = torch.zeros((2, 32, 4096), dtype=torch.uint8, device=cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    with pytest.raises(RuntimeError, match="scatter batch: destination id 5"):
        pool.make_batch([[1, 5, 2], [5]], check_unique=True)
    batch = pool.make_batch([[1, 5, 2], [5]])
    staging, _ = pool.gather(batch)
    pool.check()
    bk.set_tuning(debug_unique=1)
    pool.gather(batch, staging)                      # duplicates are fine in a gather
    with pytest.raises(RuntimeError, match=r"destination id 5 is named more than once \(entries 1 and 3\)"):
        pool.scatter(batch, staging)
    ok = pool.make_batch([[1, 5, 2], [7]], check_unique=True)
    pool.scatter(ok, staging)
    pool.check()
    bk.set_tuning(debug_unique=0)
    # the layout change's load has the same rule for its block ids
    layers = [torch.zeros((8 * 16, 2, 2, 64), dtype=torch.float16, device=cuda) for _ in range(2)]
    nhd = bk.NHDPool.from_token_kv_layers(layers, 16)
    tm = torch.zeros((2, 16, 64, 2, 2, 2), dtype=torch.float16, device=cuda)
    ids = torch.tensor([3, 3], dtype=torch.int64, device=cuda)
    with pytest.raises(RuntimeError, match="block ids: destination id 3"):
        nhd.load_token_major(tm, ids, check_unique=True)
    bk.set_tuning(debug_unique=1)
    with pytest.raises(RuntimeError, match="destination id 3"):
        nhd.load_token_major(tm, ids)
    nhd.store_token_major(tm, torch.tensor([3, 4], dtype=torch.int64, device=cuda))
    nhd.check()


def test_device_alloc_builds_a_pool_out_of_chunks_from_both_halves(bk, oracle, cuda, lib):
    """bikv_device_alloc: memory made of physical chunks mapped into one range behaves like any device
    memory — torch writes it, the movers gather from and scatter into it against the oracle — and its
    bookkeeping adds up. (Whether the probe finds a second half depends on what else the GPU holds; the
    test only requires that the allocation is complete and correct.)"""
    import ctypes as C
    from bikv_pagecopy import _lib
    _announce("device allocator")
    n_planes, n_pages, tile = 6, 9000, 16384                         # 885 MB: four chunks of 256 MiB
    nbytes = n_planes * n_pages * tile
    for spread in (True, False):
        buf = bk.DeviceBuffer(nbytes, cuda, spread=spread)
        info = buf.info
        assert info["bytes"] >= nbytes and info["bytes"] % info["chunk_bytes"] == 0
        assert info["n_chunks"] * info["chunk_bytes"] == info["bytes"] and info["chunk_bytes"] >= 256 << 20
        assert 0 <= info["n_other_half"] <= info["n_chunks"] and info["seconds"] > 0
        if not spread:
            assert info["n_other_half"] == 0 and info["n_fillers"] == 0 and info["pair_ms_same"] == 0
        else:
            assert info["pair_ms_same"] > 0       # every candidate was probed as a pair with the first chunk
        t = buf.tensor
        assert t.numel() == nbytes and t.dtype == torch.uint8 and t.device == cuda
        rng = np.random.default_rng(401)
        # the pages next to a chunk boundary are among the ones used: the pool is [planes, pages, tile] flat in
        # memory, so boundary b falls on page (b * tiles_per_chunk) % n_pages of some plane
        per_chunk = info["chunk_bytes"] // tile
        edge = [(b * per_chunk) % n_pages for b in range(1, info["n_chunks"])]
        edge = [p for e in edge for p in (e - 1, e) if 0 <= p < n_pages]
        ids_all = np.unique(np.concatenate([np.arange(8), edge, rng.integers(0, n_pages, size=52)]))
        assert ids_all.max() < n_pages and ids_all.min() >= 0
        pool_h = rng.integers(0, 256, size=(n_planes, len(ids_all), tile), dtype=np.uint8)
        pool_t = t.view(n_planes, n_pages, tile)
        pool_t.zero_()
        pool_t[:, torch.from_numpy(ids_all).to(cuda)] = torch.from_numpy(pool_h[:, : len(ids_all)]).to(cuda)
        pool = bk.PagedKVPool.from_stacked(pool_t, plane_dims=1)
        others = np.setdiff1d(ids_all, edge)
        reqs = [np.concatenate([edge, others[rng.permutation(len(others))[: 20 - len(edge)]]]).astype(np.int64), ids_all[:7]]
        assert len(reqs[0]) == 20
        batch = pool.make_batch(reqs)
        st, _ = pool.gather(batch)
        pool.check()
        pos = {int(p): i for i, p in enumerate(ids_all)}
        want = np.concatenate([np.stack([pool_h[q, [pos[int(p)] for p in r]] for q in range(n_planes)]).reshape(-1) for r in reqs])
        assert _to_np(st).tobytes() == want.tobytes(), spread
        # scatter into pages that were zero, read back with torch
        fresh = np.setdiff1d(np.arange(n_pages), ids_all)[:27]
        sb = pool.make_batch([fresh[:20], fresh[20:27]], check_unique=True)
        pool.scatter(sb, st)
        pool.check()
        got = pool_t[:, torch.from_numpy(fresh).to(cuda)].cpu().numpy()
        assert got.tobytes() == np.stack([pool_h[q, [pos[int(p)] for p in np.concatenate(reqs)]] for q in range(n_planes)]).tobytes()
        pool.close()
        del pool_t, t, st
        buf.free()
        with pytest.raises(RuntimeError, match="freed"):
            buf.tensor
    # a filler budget of zero: the placement keeps what the driver hands out first and creates nothing more
    buf = bk.DeviceBuffer(nbytes, cuda, spread=True, max_filler_bytes=0)
    assert buf.info["n_fillers"] == 0 and buf.info["bytes"] >= nbytes
    buf.tensor[:4096].fill_(7)
    assert int(buf.tensor[:4096].sum().item()) == 7 * 4096
    buf.free()
    assert lib.bikv_device_free(C.c_void_p(12345)) == _lib.EINVAL
    p = C.c_void_p()
    assert lib.bikv_device_alloc(0, 0, 0, C.byref(p)) == _lib.EINVAL
    assert lib.bikv_device_alloc(0, 1 << 20, 7, C.byref(p)) == _lib.EINVAL
    # more than the device holds: refused at once, nothing created
    assert lib.bikv_device_alloc(0, 1 << 42, 0, C.byref(p)) == _lib.EHIP and not p.value
    assert b"out of device memory" in lib.bikv_last_error()


def test_torch_allocations_inside_placed_allocations_come_from_device_alloc(bk, oracle, cuda, lib):
    """The reference's own allocation code, unchanged — per-layer torch.zeros([blocks*block, 2, heads, dim]) as in
    Worker/Worker.py:74-78 — run inside bk.placed_allocations(): torch's memory pool takes each segment from
    bikv_device_alloc (the library knows the pointers), the tensors behave like any others, and the movers gather
    from and scatter into them against the oracle. A tensor allocated outside the context is torch's own."""
    import ctypes as C
    from bikv_pagecopy import _lib
    _announce("torch memory pool on bikv_device_alloc")
    P, H, D, L, blocks = 16, 2, 128, 3, 40000          # 3 layers of 312.5 MiB
    with bk.placed_allocations(cuda):
        layers_d = [torch.zeros(blocks * P, 2, H, D, dtype=torch.float16, device=cuda) for _ in range(L)]
        big = torch.empty((1 << 30) + (64 << 20), dtype=torch.uint8, device=cuda)       # above half an arena: on its own
    outside = torch.zeros(blocks * P, 2, H, D, dtype=torch.float16, device=cuda)
    info = _lib.AllocInfo()
    for t in layers_d:
        # any address inside a placed allocation names it; the three layers were carved out of one 2 GiB arena,
        # one after the other
        assert lib.bikv_device_alloc_info(C.c_void_p(t.data_ptr()), C.byref(info)) == _lib.OK, lib.bikv_last_error()
        assert info.bytes == 2 << 30 and info.n_chunks >= 2 and info.chunk_bytes >= 256 << 20
        assert int(t.abs().sum().item()) == 0
    seg = -(-layers_d[0].numel() * 2 // (2 << 20)) * (2 << 20)
    assert [t.data_ptr() - layers_d[0].data_ptr() for t in layers_d] == [0, seg, 2 * seg]
    assert lib.bikv_device_alloc_info(C.c_void_p(big.data_ptr()), C.byref(info)) == _lib.OK and info.bytes >= big.numel()
    assert not (layers_d[0].data_ptr() <= big.data_ptr() < layers_d[0].data_ptr() + (2 << 30))
    assert lib.bikv_device_alloc_info(C.c_void_p(outside.data_ptr()), C.byref(info)) == _lib.EINVAL
    del big
    rng = np.random.default_rng(977)
    used = np.unique(np.concatenate([rng.integers(0, blocks, size=60), [0, blocks - 1, (256 << 20) // (P * 2 * H * D * 2)]]))
    rows_h = rng.integers(0, 65536, size=(L, len(used), P, 2, H, D), dtype=np.uint16)
    for l in range(L):
        v = layers_d[l].view(torch.int16).view(blocks, P, 2, H, D)
        v[torch.from_numpy(used).to(cuda)] = torch.from_numpy(rows_h[l].view(np.int16)).to(cuda)
    pool = bk.PagedKVPool.from_token_kv_layers(layers_d, P)
    # the oracle works on the used blocks only, renumbered
    small = [rows_h[l].reshape(len(used) * P, 2, H, D) for l in range(L)]
    planes_h = oracle.planes_of_token_kv_layers(small, P).view(np.uint8)
    pick = rng.permutation(len(used))
    reqs_small = [pick[:25], pick[25:31], np.array([0, 0])]
    reqs = [used[r] for r in reqs_small]
    batch = pool.make_batch(reqs, "layer_major")
    st, _ = pool.gather(batch)
    pool.check()
    assert _to_np(st).tobytes() == oracle.gather_layered_c(planes_h, reqs_small, "layer_major").tobytes()
    fresh = np.setdiff1d(np.arange(blocks), used)[rng.permutation(blocks - len(used))[:33]]
    sb = pool.make_batch([fresh[:25], fresh[25:31], fresh[31:33]], "layer_major", check_unique=True)
    pool.scatter(sb, st)
    pool.check()
    moved = np.concatenate(reqs)
    for l in range(L):
        v = layers_d[l].view(torch.int16).view(blocks, P, 2, H, D)
        assert torch.equal(v[torch.from_numpy(fresh).to(cuda)], v[torch.from_numpy(moved).to(cuda)]), f"layer {l}"
    pool.close()
    del layers_d, v, st
    torch.cuda.synchronize(cuda)


# ---- several host threads -----------------------------------------------------------------------
def test_four_host_threads_move_pages_through_one_pool(bk, oracle, cuda):
    """The reference's callers are thread pools (20 gRPC workers per process, config.yml:53,60). Four host
    threads, each on its own stream with its own batches, staging buffers and host stager, gather from and
    scatter into one pool at the same time; every thread's results are checked against the oracle."""
    import threading
    _announce("four host threads on one pool")
    n_planes, n_pages, tile, n_threads, rounds = 6, 4096, 4096, 4, 12
    rng = np.random.default_rng(77)
    pool_h = _rand_pool(rng, n_planes, n_pages, tile)
    pool_d = torch.from_numpy(pool_h).to(cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    perm = rng.permutation(n_pages)
    half = n_pages // 2
    # pages [0, half) of the permutation are only read, the rest only written: each thread owns a slice of both
    per = half // n_threads
    jobs = []
    for t in range(n_threads):
        src = perm[t * per: (t + 1) * per]
        dst = perm[half + t * per: half + (t + 1) * per]
        reqs = [src[i: i + 37].astype(np.int64) for i in range(0, per, 37)]
        dreqs = [dst[i: i + 37].astype(np.int64) for i in range(0, per, 37)]
        jobs.append((reqs, dreqs))
    errors, host_images = [], [None] * n_threads

    def work(t):
        try:
            reqs, dreqs = jobs[t]
            stream = torch.cuda.Stream(cuda)
            stager = bk.HostStager(cuda, chunk_bytes=16 * tile, n_buffers=2, chunks_per_launch=2)
            with torch.cuda.stream(stream):
                gb = pool.make_batch(reqs, "layer_major")
                sb = pool.make_batch(dreqs, "layer_major", check_unique=True)
                staging, _ = pool.empty_staging(gb)
                for _ in range(rounds):
                    pool.gather(gb, staging)
                    pool.scatter(sb, staging)          # the gathered pages land in this thread's own pages
                host = bk.pinned_empty(gb.n_slots * tile)
                stager.gather_to_host(pool, gb, host, "auto")
                stream.synchronize()
            want = oracle.gather_layered_c(pool_h, reqs, "layer_major")
            if _to_np(staging).tobytes() != want.tobytes():
                errors.append(f"thread {t}: gathered image differs")
            if host.numpy().tobytes() != want.tobytes():
                errors.append(f"thread {t}: host image differs")
            host_images[t] = want
            stager.close()
        except Exception as e:                          # noqa: BLE001 - reported below
            errors.append(f"thread {t}: {type(e).__name__}: {e}")

    threads = [threading.Thread(target=work, args=(t,)) for t in range(n_threads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    torch.cuda.synchronize(cuda)
    pool.check()
    assert not errors, errors
    for t in range(n_threads):
        oracle.scatter_layered_c(pool_h, jobs[t][1], host_images[t], "layer_major")
    assert _to_np(pool_d).tobytes() == pool_h.tobytes()
