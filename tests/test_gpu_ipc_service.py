"""The `ipc_service` drop-in on a real GPU: the reference's two scripted scenarios
(Bi-KV/SharedMemory/CUDA_Shared/test_page_ipc.py, test_zero_copy.py) with producer and consumer in
one process, seeded-data variants of them (the constant-7 data of the originals cannot detect a
wrong offset), producer_send / consumer_receive, ring wrap-around and the error paths."""
import json
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture()
def ipc(lib, cuda):
    import ipc_service
    ipc_service.producer_cleanup()
    ipc_service.consumer_cleanup()
    yield ipc_service
    ipc_service.producer_cleanup()
    ipc_service.consumer_cleanup()


def _dims(ipc, s, total_tokens):
    d = ipc.TensorDims()
    d.total_tokens = total_tokens
    d.head_size, d.num_kv_heads, d.num_layers, d.kv_pair = s["head_size"], s["num_kv_heads"], s["num_layers"], s["kv_pair"]
    return d


def _scenario(name):
    """The reference's scripted scenario. Its ring is 2 GiB; a ring that size is never exported over HIP
    IPC here, so the scenario runs on a ring 4 KiB short of it, which holds the same 7 transfers and
    wraps at the same points."""
    with open(os.path.join(GOLDEN, "reference_scenarios.json")) as f:
        s = json.load(f)[name]
    s["buffer_size"] = min(s["buffer_size"], (2 << 30) - 4096)
    return s


def test_reference_page_ipc_scenario(ipc, cuda):
    """200 pages x 50 tokens of 7s, identity offsets, 2 GiB ring, 10 transfers: dim 5, shape
    (10000,128,2,28,2), all 7 (test_page_ipc.py:127-150); and the ring advances by 273.4 MiB per
    transfer and restarts at 0 when the next batch would not fit."""
    s = _scenario("test_page_ipc")
    print("[case] reference test_page_ipc scenario", flush=True)
    name = f"/bikv_test_page_ipc_{os.getpid()}"
    ipc.consumer_init(0, name, s["buffer_size"])
    ipc.producer_init(0, name.encode())       # callers pass bytes (kvcache.py:72) or str (the scripts)
    ept = s["head_size"] * s["num_kv_heads"] * s["num_layers"] * s["kv_pair"]
    page_elements = s["page_size"] * ept
    n = s["num_pages"]
    cache = torch.full((n, s["page_size"], s["head_size"], s["num_kv_heads"], s["num_layers"], s["kv_pair"]),
                       s["fill_value"], dtype=torch.float16, device=cuda)
    offs = torch.tensor([i * page_elements for i in range(n)], dtype=torch.int64, device=cuda)
    dims = _dims(ipc, s, n * s["page_size"])
    per = n * page_elements * 2
    ptrs = []
    for k in range(s["num_transfers"] - 1):
        ipc.producer_copy_pages(cache, offs, offs, s["page_size"], dims)
        result = ipc.consumer_receive()
        assert result.dim() == s["expected_dim"]
        assert tuple(result.shape) == tuple(s["expected_shape"])
        assert result.dtype == torch.float16 and result.device == cuda
        assert torch.allclose(result, torch.full_like(result, s["expected_value"]))
        ptrs.append(result.data_ptr())
    fit = s["buffer_size"] // per            # 7 transfers fit a 2 GiB ring
    base = ptrs[0]
    assert [p - base for p in ptrs] == [(k % fit) * per for k in range(len(ptrs))]


def test_reference_zero_copy_scenario(ipc, cuda):
    s = _scenario("test_zero_copy")
    print("[case] reference test_zero_copy scenario", flush=True)
    name = f"/bikv_test_zero_copy_{os.getpid()}"
    ipc.consumer_init(0, name, s["buffer_size"])
    ipc.producer_init(0, name)
    ept = s["head_size"] * s["num_kv_heads"] * s["num_layers"] * s["kv_pair"]
    page_elements = s["page_size"] * ept
    n = s["num_pages"]
    cpu_data = torch.full((n * page_elements,), s["fill_value"], dtype=torch.float16).pin_memory()
    page_indices = torch.arange(n, dtype=torch.int64, device=cuda)
    dest = torch.arange(0, n * page_elements, page_elements, dtype=torch.int64, device=cuda)
    dims = _dims(ipc, s, n * s["page_size"])
    for _ in range(3):
        ipc.producer_zero_copy_pages(cpu_data, page_indices, dest, s["page_size"], dims)
        t = ipc.consumer_receive()
        assert tuple(t.shape) == tuple(s["expected_shape"])
        assert torch.all(t == s["expected_value"])
        assert t.is_cuda


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.uint8])
def test_copy_pages_seeded_data_against_oracle(ipc, oracle, cuda, dtype):
    """Random data, shuffled page order, duplicate source pages: what constant data cannot check."""
    print(f"[case] producer_copy_pages seeded {dtype}", flush=True)
    name = f"/bikv_test_seeded_{os.getpid()}"
    d = ipc.TensorDims()
    d.head_size, d.num_kv_heads, d.num_layers, d.kv_pair = 64, 2, 3, 2
    page_size, pool_pages, n = 16, 40, 23
    page_elements = page_size * 64 * 2 * 3 * 2
    es = torch.empty((), dtype=dtype).element_size()
    ipc.consumer_init(0, name, 3 * n * page_elements * es + 1000)
    ipc.producer_init(0, name)
    rng = np.random.default_rng(17)
    np_dt = {1: np.uint8, 2: np.uint16}[es]
    pool_h = rng.integers(0, 256, size=pool_pages * page_elements * es, dtype=np.uint8).view(np_dt)
    pool_d = torch.from_numpy(pool_h.view(np.uint8)).to(cuda).view(dtype)
    for step in range(4):                                   # the 4th transfer wraps
        ids = rng.integers(0, pool_pages, size=n)
        so = ids * page_elements
        do = rng.permutation(n).astype(np.int64) * page_elements
        ipc.producer_copy_pages(pool_d, torch.from_numpy(so).to(cuda), torch.from_numpy(do).to(cuda), page_size, d)
        got = ipc.consumer_receive(timeout_ms=5000)
        assert got.dtype == dtype and tuple(got.shape) == (n * page_size, 64, 2, 3, 2)
        want = np.zeros(n * page_elements, dtype=np_dt)
        oracle.copy_runs_c(pool_h, want, so, do, page_elements)
        assert got.cpu().contiguous().view(torch.uint8).numpy().tobytes() == want.tobytes()
    from bikv_pagecopy import _lib
    ctrl = _lib.load().bikv_consumer_control().contents
    ring = oracle.Ring(buffer_size=ctrl.buffer_size)
    for step in range(4):
        oracle.ring_step_c(ring, n, page_size, (64, 2, 3, 2), es)
    assert (ctrl.current_offset, ctrl.last_valid_offset, ctrl.data_size, ctrl.tensor_dim) == \
        (ring.current_offset, ring.last_valid_offset, ring.data_size, ring.tensor_dim)
    assert list(ctrl.tensor_shape) == list(ring.tensor_shape)


def test_producer_send_round_trip(ipc, oracle, cuda):
    print("[case] producer_send / consumer_receive", flush=True)
    name = f"/bikv_test_send_{os.getpid()}"
    ipc.consumer_init(0, name, 1 << 20)
    ipc.producer_init(0, name)
    ring = oracle.Ring(buffer_size=1 << 20)
    base = None
    for shape in [(1000, 128), (7, 5, 3, 2, 4), (300000,), (300000,), (2, 3)]:
        t = torch.randn(shape, device=cuda).to(torch.float16)
        ipc.producer_send(t)
        r = ipc.consumer_receive(timeout_ms=5000)
        assert r.shape == t.shape and r.dtype == torch.float16 and torch.equal(r, t)
        at = oracle.ring_send_c(ring, t.numel() * 2, list(shape))
        base = base if base is not None else r.data_ptr() - at
        assert r.data_ptr() - base == at            # same wrap rule as the reference
    with pytest.raises(RuntimeError, match="float16"):
        ipc.producer_send(torch.zeros(4, device=cuda))
    with pytest.raises(RuntimeError, match="contiguous"):
        ipc.producer_send(torch.zeros(4, 4, dtype=torch.float16, device=cuda).t())
    with pytest.raises(RuntimeError, match="CUDA"):
        ipc.producer_send(torch.zeros(4, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="does not fit"):
        ipc.producer_send(torch.zeros(1 << 20, dtype=torch.float16, device=cuda))


def test_error_paths(ipc, cuda):
    print("[case] ipc_service error paths", flush=True)
    name = f"/bikv_test_err_{os.getpid()}"
    d = ipc.TensorDims()
    d.head_size, d.num_kv_heads, d.num_layers, d.kv_pair = 8, 1, 1, 2
    off = torch.zeros(2, dtype=torch.int64, device=cuda)
    data = torch.zeros(1024, dtype=torch.float16, device=cuda)
    with pytest.raises(RuntimeError, match="not initialised"):
        ipc.producer_copy_pages(data, off, off, 4, d)
    with pytest.raises(RuntimeError, match="not initialised"):
        ipc.consumer_receive(timeout_ms=10)
    ipc.consumer_init(0, name, 4096)
    with pytest.raises(RuntimeError, match="already initialised"):
        ipc.consumer_init(0, name, 4096)
    ipc.producer_init(0, name)
    with pytest.raises(RuntimeError, match="timed out"):
        ipc.consumer_receive(timeout_ms=50)             # nothing was produced
    with pytest.raises(RuntimeError, match="Cache data must be on CUDA"):
        ipc.producer_copy_pages(data.cpu(), off, off, 4, d)
    with pytest.raises(RuntimeError, match="Cache data must be contiguous"):
        ipc.producer_copy_pages(data[::2], off, off, 4, d)
    with pytest.raises(RuntimeError, match="CPU data must be pinned memory"):
        ipc.producer_zero_copy_pages(data.cpu(), off, off, 4, d)
    with pytest.raises(RuntimeError, match="Page indices must be on CUDA"):
        ipc.producer_zero_copy_pages(data.cpu().pin_memory(), off.cpu(), off, 4, d)
    with pytest.raises(RuntimeError, match="does not fit"):
        ipc.producer_copy_pages(data, torch.zeros(64, dtype=torch.int64, device=cuda),
                                torch.zeros(64, dtype=torch.int64, device=cuda), 4, d)
    bad = torch.tensor([0, 100000], dtype=torch.int64, device=cuda)
    with pytest.raises(RuntimeError, match="source-range"):
        ipc.producer_copy_pages(data, bad, torch.tensor([0, 64], dtype=torch.int64, device=cuda), 4, d)
    # nothing was published by the failed calls
    with pytest.raises(RuntimeError, match="timed out"):
        ipc.consumer_receive(timeout_ms=50)
    ipc.consumer_cleanup()
    assert not os.path.exists("/dev/shm" + name)        # the consumer unlinks its object


@pytest.mark.parametrize("pinned_host_pool", [False, True])
def test_cache_side_callers_from_task_info(ipc, oracle, cuda, pinned_host_pool):
    """KVCache.shared_data_batch_pages / _cpu2gpu (kvcache.py:132-366) as functions: the coordinator's
    task info in, pages in the consumer's ring out."""
    from bikv_pagecopy import kvcache_calls
    print(f"[case] cache-side callers, pinned host pool={pinned_host_pool}", flush=True)
    name = f"/bikv_test_callers_{os.getpid()}"
    dims, page_size, pool_pages = (64, 2, 3, 2), 16, 50
    ept = dims[0] * dims[1] * dims[2] * dims[3]
    page_elems = page_size * ept
    ipc.consumer_init(0, name, 64 << 20)
    ipc.producer_init(0, name)
    rng = np.random.default_rng(23)
    pool_h = rng.integers(0, 65536, size=pool_pages * page_elems, dtype=np.uint16)
    pool_t = torch.from_numpy(pool_h.view(np.int16)).view(torch.float16)
    pool_t = pool_t.pin_memory() if pinned_host_pool else pool_t.to(cuda)
    info = {"infer_worker": 0, "token_num": 40 + 16 + 33,
            "id_token_pair": [(11, 40), (12, 16), (13, 33)],            # 3, 1 and 3 pages of 16 tokens
            "cache_pages_list": [[7, 2, 49], [4], [30, 31, 0]]}
    if pinned_host_pool:
        n, tokens = kvcache_calls.shared_data_batch_pages_cpu2gpu(pool_t, info, page_size, cuda, dims)
    else:
        n, tokens = kvcache_calls.shared_data_batch_pages(pool_t, info, page_size, dims)
    assert (n, tokens) == (7, 7 * page_size)
    # the per-stage timers the reference prints under SM_DEBUG (kvcache.py:155-238)
    t = kvcache_calls.last_stage_times()
    assert (t.pages, t.tokens, t.data_bytes) == (7, 7 * page_size, 7 * page_elems * 2)
    assert t.index_ms > 0 and t.upload_ms > 0 and t.copy_ms > 0 and t.total_ms >= t.copy_ms
    assert t.copy_MBps == pytest.approx(t.data_bytes / (t.copy_ms * 1e-3) / 2 ** 20)
    assert "IPC page copy" in t.report() and "MB/s" in t.report()
    got = ipc.consumer_receive(timeout_ms=5000)
    assert tuple(got.shape) == (7 * page_size,) + dims
    pages = np.array([7, 2, 49, 4, 30, 31, 0])
    want = np.zeros(7 * page_elems, dtype=np.uint16)
    oracle.copy_runs_c(pool_h, want, pages * page_elems, np.arange(7) * page_elems, page_elems)
    assert got.cpu().contiguous().view(torch.int16).numpy().tobytes() == want.tobytes()
    # the reference's literal (packed) destination offsets, for the record
    so, do, total = oracle.build_offsets_loops(info["cache_pages_list"], info["id_token_pair"], page_size, ept)
    assert total == 89 and do[3] == 40 * ept and so[2] == 49 * page_elems
    with pytest.raises(RuntimeError):
        kvcache_calls.shared_data_batch_pages(pool_t.cpu() if not pinned_host_pool else pool_t, info, page_size, dims)


@pytest.mark.parametrize("pinned_host_pool", [False, True])
def test_cache_side_callers_pack_partial_pages_exactly(ipc, oracle, cuda, pinned_host_pool):
    """Packed transfer: the consumer receives each item's tokens, cut to its token count, back to
    back (what kvcache.py:161-174's destination offsets describe), not whole pages."""
    from bikv_pagecopy import kvcache_calls
    print(f"[case] exact packing, pinned host pool={pinned_host_pool}", flush=True)
    name = f"/bikv_test_packed_{os.getpid()}"
    dims, page_size, pool_pages = (64, 2, 3, 2), 16, 50
    ept = dims[0] * dims[1] * dims[2] * dims[3]
    ipc.consumer_init(0, name, 64 << 20)
    ipc.producer_init(0, name)
    try:
        rng = np.random.default_rng(29)
        pool_h = rng.integers(0, 65536, size=(pool_pages * page_size, ept), dtype=np.uint16)
        pool_t = torch.from_numpy(pool_h.view(np.int16)).view(torch.float16)
        pool_t = pool_t.pin_memory() if pinned_host_pool else pool_t.to(cuda)
        pages_list = [[7, 2, 49], [4], [], [30, 31, 0], [5]]
        tokens = [40, 16, 0, 33, 1]
        info = {"infer_worker": 0, "token_num": sum(tokens),
                "id_token_pair": [(10 + i, t) for i, t in enumerate(tokens)], "cache_pages_list": pages_list}
        if pinned_host_pool:
            n, total = kvcache_calls.shared_data_batch_pages_cpu2gpu(pool_t, info, page_size, cuda, dims, "exact")
        else:
            n, total = kvcache_calls.shared_data_batch_pages(pool_t, info, page_size, dims, "exact")
        assert (n, total) == (8, 90)
        got = ipc.consumer_receive(timeout_ms=5000)
        assert tuple(got.shape) == (90,) + dims
        want = oracle.packed_items_np(pool_h, pages_list, tokens, page_size)
        assert got.cpu().contiguous().view(torch.int16).numpy().tobytes() == want.tobytes()
        # a total that is too small makes the last run leave the published window: reported, not written
        d = ipc.TensorDims()
        d.total_tokens, d.head_size, d.num_kv_heads, d.num_layers, d.kv_pair = (20,) + dims
        t = lambda a: torch.tensor(a, dtype=torch.int64, device=cuda)
        with pytest.raises(RuntimeError, match="destination-range"):
            ipc.producer_copy_tokens(pool_t, t([0, 16]), t([0, 16]), t([16, 16]), page_size, d)
    finally:
        ipc.producer_cleanup()
        ipc.consumer_cleanup()


def test_backpressure_holds_the_producer_until_release(ipc, cuda):
    """sem_complete in use. With back-pressure on, the producer copies ahead into free ring space but
    publishes only after the consumer released the previous tensor, and never copies over a held one."""
    print("[case] ring back-pressure", flush=True)
    name = f"/bikv_test_bp_{os.getpid()}"
    n = 1 << 16
    ipc.consumer_init(0, name, 5 * n * 2 // 2)          # 2.5 tensors of n fp16
    ipc.producer_init(0, name)
    try:
        ipc.producer_set_backpressure(True, timeout_ms=200)
        tensors = [torch.full((n,), float(i + 1), dtype=torch.float16, device=cuda) for i in range(3)]
        big = torch.full((2 * n,), 9.0, dtype=torch.float16, device=cuda)
        ctrl = ipc._lib.load().bikv_producer_control().contents
        ipc.producer_send(tensors[0])
        first = ipc.consumer_receive(timeout_ms=5000)
        with pytest.raises(RuntimeError, match="release the previous transfer"):
            ipc.producer_send(tensors[1])               # copied behind `first`, but not published
        assert (ctrl.last_valid_offset, ctrl.data_size) == (0, n * 2) and bool((first == 1).all())
        with pytest.raises(RuntimeError, match="timed out"):
            ipc.consumer_receive(timeout_ms=50)         # nothing new to receive
        ipc.consumer_release()
        ipc.producer_send(tensors[1])
        second = ipc.consumer_receive(timeout_ms=5000)
        assert second.data_ptr() == first.data_ptr() + n * 2 and bool((second == 2).all())
        # a transfer of 2n elements has to wrap to offset 0 and would reach into `second`: the producer
        # blocks BEFORE copying
        with pytest.raises(RuntimeError, match="release the ring space"):
            ipc.producer_send(big)
        torch.cuda.synchronize()
        assert bool((second == 2).all())
        ipc.consumer_release()
        ipc.producer_send(big)
        third = ipc.consumer_receive(timeout_ms=5000)
        assert third.data_ptr() == first.data_ptr() and third.numel() == 2 * n and bool((third == 9).all())
        ipc.consumer_release()
        ipc.producer_send(tensors[2])                   # 2n + n > 2.5n: wraps again
        fourth = ipc.consumer_receive(timeout_ms=5000)
        assert fourth.data_ptr() == first.data_ptr() and bool((fourth == 3).all())
        # switched off again: the reference's behaviour (publishes without asking)
        ipc.producer_set_backpressure(False)
        ipc.producer_send(tensors[0])
        ipc.producer_send(tensors[1])
        assert ipc.consumer_receive(timeout_ms=5000) is not None
    finally:
        ipc.producer_cleanup()
        ipc.consumer_cleanup()
    with pytest.raises(RuntimeError, match="not initialised"):
        ipc.consumer_release()
    with pytest.raises(RuntimeError, match="not initialised"):
        ipc.producer_set_backpressure(True)


def test_persistent_index_buffers_for_offsets_and_batches(ipc, oracle, cuda):
    """RunIndexPool = the reference's src_index_pool / dst_index_pool (kvcache.py:60-64): tables of
    successive transfers reuse the same device buffers."""
    import bikv_pagecopy as bk
    from bikv_pagecopy import kvcache_calls
    print("[case] persistent index buffers", flush=True)
    name = f"/bikv_test_idxpool_{os.getpid()}"
    dims, page_size, pool_pages = (64, 2, 3, 2), 16, 50
    ept = dims[0] * dims[1] * dims[2] * dims[3]
    ipc.consumer_init(0, name, 64 << 20)
    ipc.producer_init(0, name)
    rng = np.random.default_rng(31)
    pool_h = rng.integers(0, 65536, size=(pool_pages * page_size, ept), dtype=np.uint16)
    pool_t = torch.from_numpy(pool_h.view(np.int16)).view(torch.float16).to(cuda)
    idx = bk.RunIndexPool(max_pages=pool_pages, device=cuda)
    base = idx.dev.data_ptr()
    for pages_list, tokens in (([[7, 2, 49], [4]], [40, 16]), ([[1], [30, 31, 0, 9], [5, 6]], [3, 64, 17])):
        info = {"infer_worker": 0, "token_num": sum(tokens),
                "id_token_pair": list(enumerate(tokens)), "cache_pages_list": pages_list}
        n, total = kvcache_calls.shared_data_batch_pages(pool_t, info, page_size, dims, "exact", index_pool=idx)
        got = ipc.consumer_receive(timeout_ms=5000)
        want = oracle.packed_items_np(pool_h, pages_list, tokens, page_size)
        assert total == sum(tokens) and got.cpu().contiguous().view(torch.int16).numpy().tobytes() == want.tobytes()
        assert idx.dev.data_ptr() == base
    with pytest.raises(RuntimeError, match="exceeds pool size"):
        idx.load(np.zeros((2, pool_pages + 1), dtype=np.int64))
    # the layered batch builder takes the same kind of pool
    planes_h = rng.integers(0, 256, size=(4, 30, 4096), dtype=np.uint8)
    kv = bk.PagedKVPool.from_stacked(torch.from_numpy(planes_h).to(cuda), plane_dims=1)
    bidx = bk.RunIndexPool(max_pages=64, device=cuda)
    for reqs in ([rng.permutation(30)[:11], rng.permutation(30)[:5]], [rng.permutation(30)[:20]]):
        for layout in ("layer_major", "page_major"):
            b = kv.make_batch(reqs, layout, index_pool=bidx)
            st, _ = kv.gather(b)
            kv.check()
            assert st.cpu().numpy().tobytes() == oracle.gather_layered_c(planes_h, reqs, layout).tobytes()


@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
def test_layered_gather_straight_into_the_ring(ipc, oracle, cuda, layout):
    """The staging image of a layered gather IS the consumer's ring window (what a transfer between
    two GPUs does with a peer-mapped buffer): reserve, gather into the window, publish."""
    import bikv_pagecopy as bk
    print(f"[case] layered gather into the ring, {layout}", flush=True)
    name = f"/bikv_test_ringgather_{os.getpid()}"
    rng = np.random.default_rng(37)
    n_planes, n_pages, P, H, D = 6, 48, 16, 2, 64
    tile = P * H * D * 2
    pool_h = rng.integers(0, 256, size=(n_planes, n_pages, tile), dtype=np.uint8)
    pool = bk.PagedKVPool.from_stacked(torch.from_numpy(pool_h).to(cuda), plane_dims=1)
    ipc.consumer_init(0, name, int(2.5 * 20 * n_planes * tile))
    ipc.producer_init(0, name)
    ctrl = ipc._lib.load().bikv_producer_control().contents
    offsets = []
    for k in range(4):                                      # the fourth transfer wraps
        reqs = [rng.permutation(n_pages)[:11], rng.permutation(n_pages)[:9]]
        batch = pool.make_batch(reqs, layout)
        window = ipc.producer_reserve(batch.n_slots * tile)
        pool.gather(batch, window)
        shape = (n_planes, 20, P, H, D) if layout == "layer_major" else (20, n_planes, P, H, D)
        ipc.producer_publish(shape, torch.float16)
        offsets.append(int(ctrl.last_valid_offset))
        got = ipc.consumer_receive(timeout_ms=5000)
        assert tuple(got.shape) == shape and got.dtype == torch.float16
        assert got.cpu().contiguous().view(torch.uint8).numpy().tobytes() == oracle.gather_layered_c(pool_h, reqs, layout).tobytes(), k
    per = 20 * n_planes * tile
    assert offsets == [0, per, 0, per]
    # a kernel that skipped work is not published
    bad = pool.make_batch([[1, 2, 3]], layout)
    bad.index[0, 1] = n_pages + 7
    before = (int(ctrl.last_valid_offset), int(ctrl.current_offset))
    window = ipc.producer_reserve(bad.n_slots * tile)
    pool.gather(bad, window)
    with pytest.raises(RuntimeError, match="page-id"):
        ipc.producer_publish((3 * n_planes, P, H, D), torch.float16)
    assert (int(ctrl.last_valid_offset), int(ctrl.current_offset)) == before
    with pytest.raises(RuntimeError, match="timed out"):
        ipc.consumer_receive(timeout_ms=50)
    with pytest.raises(RuntimeError, match="does not fit"):
        ipc.producer_reserve(1 << 40)


def test_nothing_else_may_use_the_ring_while_a_window_is_reserved(ipc, cuda):
    """Between reserve and publish the write offset belongs to the reservation: send, copy_pages,
    copy_tokens and a second reserve would be handed the same bytes, so they are refused; the
    reservation is published at the offset it was given, or given up with producer_cancel."""
    print("[case] reserve / publish misuse", flush=True)
    name = f"/bikv_test_reserve_misuse_{os.getpid()}"
    ipc.consumer_init(0, name, 1 << 20)
    ipc.producer_init(0, name)
    ctrl = ipc._lib.load().bikv_producer_control().contents
    first = torch.arange(4096, dtype=torch.float16, device=cuda)
    ipc.producer_send(first)                                   # ring offset 0..8192
    assert ipc.consumer_receive(timeout_ms=5000).data_ptr() == ipc._lib.load().bikv_consumer_buffer()
    window = ipc.producer_reserve(2048)
    window.copy_(torch.arange(2048, device=cuda).to(torch.uint8))
    d = ipc.TensorDims()
    d.head_size, d.num_kv_heads, d.num_layers, d.kv_pair = 8, 1, 1, 2
    offs = torch.zeros(1, dtype=torch.int64, device=cuda)
    for misuse in (lambda: ipc.producer_send(first),
                   lambda: ipc.producer_copy_pages(first, offs, offs, 16, d),
                   lambda: ipc.producer_copy_tokens(first, offs, offs, torch.ones(1, dtype=torch.int64, device=cuda), 16, d),
                   lambda: ipc.producer_reserve(64)):
        with pytest.raises(RuntimeError, match="reserved ring window"):
            misuse()
    assert int(ctrl.current_offset) == 8192                    # untouched by the refused calls
    ipc.producer_publish((2048,), torch.uint8)
    assert (int(ctrl.last_valid_offset), int(ctrl.current_offset), int(ctrl.data_size)) == (8192, 8192 + 2048, 2048)
    got = ipc.consumer_receive(timeout_ms=5000)
    assert torch.equal(got, torch.arange(2048, device=cuda).to(torch.uint8))
    # a reservation that is given up leaves the ring where it was
    ipc.producer_reserve(512)
    ipc.producer_cancel()
    ipc.producer_send(first)
    assert int(ctrl.last_valid_offset) == 8192 + 2048
    with pytest.raises(RuntimeError, match="nothing is reserved"):
        ipc.producer_publish((1,), torch.uint8)


def test_whole_page_copy_cannot_write_past_the_published_tensor(ipc, cuda):
    """A destination offset beyond the transfer's own bytes is skipped and reported even though the ring
    has room behind it: those bytes may belong to a tensor the consumer still holds."""
    print("[case] copy_pages destination extent", flush=True)
    name = f"/bikv_test_dst_extent_{os.getpid()}"
    ipc.consumer_init(0, name, 1 << 20)
    ipc.producer_init(0, name)
    d = ipc.TensorDims()
    d.head_size, d.num_kv_heads, d.num_layers, d.kv_pair = 8, 1, 1, 2
    page_size, page_elems = 4, 4 * 16
    pool = torch.arange(8 * page_elems, dtype=torch.float16, device=cuda)
    so = torch.tensor([0, page_elems], dtype=torch.int64, device=cuda)
    do = torch.tensor([0, 2 * page_elems], dtype=torch.int64, device=cuda)   # second run lands one page too far
    with pytest.raises(RuntimeError, match="destination-range"):
        ipc.producer_copy_pages(pool, so, do, page_size, d)
    with pytest.raises(RuntimeError, match="timed out"):
        ipc.consumer_receive(timeout_ms=50)
    # a flag raised by somebody else's unchecked launch does not fail the producer's next transfer
    import bikv_pagecopy as bk
    bk.copy_runs(pool, torch.empty_like(pool), torch.tensor([1 << 40], dtype=torch.int64, device=cuda),
                 torch.zeros(1, dtype=torch.int64, device=cuda), page_elems)
    ipc.producer_copy_pages(pool, so, torch.tensor([0, page_elems], dtype=torch.int64, device=cuda), page_size, d)
    assert tuple(ipc.consumer_receive(timeout_ms=5000).shape) == (8, 8, 1, 1, 2)
    from bikv_pagecopy import runs
    with pytest.raises(RuntimeError, match="source-range"):
        runs.check(cuda)                                       # ... and is still there for its owner


def test_a_ring_of_2_gib_is_not_exported_over_ipc(ipc, cuda):
    """The consumer leaves the IPC handle of a ring of 2 GiB or more zeroed; a producer in the same
    process still works on it."""
    print("[case] 2 GiB ring stays in-process", flush=True)
    name = f"/bikv_test_bigring_local_{os.getpid()}"
    ipc.consumer_init(0, name, 2 << 30)
    ctrl = ipc._lib.load().bikv_consumer_control().contents
    assert bytes(ctrl.ipc_handle) == bytes(64)
    ipc.producer_init(0, name)
    t = torch.arange(1000, dtype=torch.float16, device=cuda)
    ipc.producer_send(t)
    assert torch.equal(ipc.consumer_receive(timeout_ms=5000), t)
    ipc.producer_cleanup()
    ipc.consumer_cleanup()
    ipc.consumer_init(0, name, 1 << 20)
    assert bytes(ipc._lib.load().bikv_consumer_control().contents.ipc_handle) != bytes(64)


def test_packed_transfer_against_committed_digest(ipc, cuda):
    """The token-exact packed transfer against tests/golden/packed_and_layout.json (no oracle in the loop)."""
    import hashlib
    import importlib.util
    import json
    from bikv_pagecopy import kvcache_calls
    print("[case] packed transfer golden digest", flush=True)
    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(golden, "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    with open(os.path.join(golden, "packed_and_layout.json")) as f:
        e = json.load(f)["packed_transfer"]
    pool, pages_list, tokens, page_size = mg.packed_case()
    dims = (12, 1, 1, 2)                                     # 24 elements per token
    name = f"/bikv_test_goldpack_{os.getpid()}"
    ipc.consumer_init(0, name, 8 << 20)
    ipc.producer_init(0, name)
    pool_d = torch.from_numpy(pool.view(np.int16)).view(torch.float16).to(cuda)
    info = {"infer_worker": 0, "token_num": sum(tokens), "id_token_pair": list(enumerate(tokens)),
            "cache_pages_list": pages_list}
    n, total = kvcache_calls.shared_data_batch_pages(pool_d, info, page_size, dims, "exact")
    got = ipc.consumer_receive(timeout_ms=5000)
    assert total == e["total_tokens"] and tuple(got.shape) == (total,) + dims
    digest = hashlib.sha256(got.cpu().contiguous().view(torch.int16).numpy().tobytes()).hexdigest()
    assert digest == e["received_sha256"]


def test_three_producer_threads_share_the_ring_without_losing_a_transfer(ipc, cuda):
    """The reference's callers are gRPC thread pools over process-global ring state (ipc_service.cpp:9-17).
    Here three threads call producer_send / producer_copy_pages at once, with back-pressure on, while a
    fourth receives: every transfer arrives exactly once, whole, and carries its own sender's bytes — no
    window handed out twice, no publication lost."""
    import threading
    print("[case] three producer threads, one ring", flush=True)
    name = f"/bikv_test_threads_{os.getpid()}"
    n_threads, per_thread, n = 3, 40, 1 << 14
    ipc.consumer_init(0, name, 5 * n * 2 // 2)          # 2.5 tensors of n fp16: the ring wraps all the time
    ipc.producer_init(0, name)
    errors, seen = [], []

    def consume():
        try:
            for _ in range(n_threads * per_thread):
                t = ipc.consumer_receive(timeout_ms=15000)
                vals = t.reshape(-1).view(torch.int16).cpu()
                tag = int(vals[0].item())
                if not bool((vals == tag).all()) or t.numel() != n:
                    errors.append(f"mixed or short transfer (tag {tag})")
                seen.append(tag)
                ipc.consumer_release()
        except Exception as e:  # noqa: BLE001
            errors.append(f"consumer: {e}")

    def produce(tid):
        try:
            torch.cuda.set_device(cuda)
            stream = torch.cuda.Stream(device=cuda)
            d = ipc.TensorDims()
            d.head_size, d.num_kv_heads, d.num_layers, d.kv_pair = 64, 2, 1, 2
            page_elems = 16 * 64 * 2 * 1 * 2
            runs = n // page_elems
            offs = torch.arange(runs, dtype=torch.int64, device=cuda) * page_elems
            with torch.cuda.stream(stream):
                for k in range(per_thread):
                    tag = tid * per_thread + k + 1
                    src = torch.full((n,), tag, dtype=torch.int16, device=cuda).view(torch.float16)
                    if k % 2:
                        ipc.producer_send(src)
                    else:
                        ipc.producer_copy_pages(src, offs, offs, 16, d)
        except Exception as e:  # noqa: BLE001
            errors.append(f"producer {tid}: {e}")

    try:
        ipc.producer_set_backpressure(True, timeout_ms=15000)
        threads = [threading.Thread(target=consume)] + [threading.Thread(target=produce, args=(t,)) for t in range(n_threads)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(120)
        assert not any(t.is_alive() for t in threads), "a thread is stuck"
        assert not errors, errors
        assert sorted(seen) == list(range(1, n_threads * per_thread + 1))
    finally:
        ipc.producer_cleanup()
        ipc.consumer_cleanup()
