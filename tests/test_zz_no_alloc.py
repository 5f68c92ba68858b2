"""The allocation-free entry point, bikv_gather_to_host_noalloc, against bikv_gather_to_host: same pool,
same batches, bit-exact, called through the C ABI; two calls in a row, the second with a smaller input
(the static scratch keeps the first call's bytes). The module name sorts last on purpose."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _call_noalloc(lib, _lib, pool, batch, host, host_scale=None, stream=None):
    d = batch.desc()
    rp = batch.req_pages.ctypes.data_as(C.POINTER(C.c_int64))
    return lib.bikv_gather_to_host_noalloc(
        pool._h, C.byref(d), rp, len(batch.req_pages), 0 if batch.layout == "layer_major" else 1,
        host.data_ptr(), host.numel(), host_scale.data_ptr() if host_scale is not None else None,
        host_scale.numel() if host_scale is not None else 0, stream)


@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
def test_noalloc_gather_matches_the_allocating_entry_point(lib, oracle, cuda, layout):
    import bikv_pagecopy as bk
    from bikv_pagecopy import _lib
    print(f"[case] allocation-free gather to host, {layout}", flush=True)
    assert lib.bikv_init(0) == _lib.OK
    rng = np.random.default_rng(71)
    # 1.25 MiB tiles: 12 tiles fill the 16 MiB scratch, so both calls below take several launches
    n_planes, n_pages, tile, stile = 5, 40, 1280 * 1024, 32
    pool_h = rng.integers(0, 256, size=(n_planes, n_pages, tile), dtype=np.uint8)
    scale_h = rng.integers(0, 256, size=(n_planes, n_pages, stile), dtype=np.uint8)
    pool = bk.PagedKVPool.from_stacked(torch.from_numpy(pool_h).to(cuda), plane_dims=1,
                                       scale=torch.from_numpy(scale_h).to(cuda))
    stager = bk.HostStager(cuda, chunk_bytes=4 << 20, n_buffers=2, chunks_per_launch=2)
    stream = C.c_void_p(torch.cuda.current_stream(cuda).cuda_stream)
    for reqs in ([rng.permutation(n_pages)[:13], rng.permutation(n_pages)[:1], rng.permutation(n_pages)[:9]],
                 [rng.permutation(n_pages)[:3]]):                      # the second call is the smaller one
        batch = pool.make_batch(reqs, layout)
        nb, ns = batch.n_slots * tile, batch.n_slots * stile
        want, swant = bk.pinned_empty(nb).fill_(0x11), bk.pinned_empty(ns).fill_(0x11)
        stager.gather_to_host(pool, batch, want, "pipelined", host_scale=swant)          # the existing entry point
        got, sgot = bk.pinned_empty(nb).fill_(0xA5), bk.pinned_empty(ns).fill_(0xA5)
        torch.cuda.current_stream(cuda).synchronize()                  # the index upload is done
        assert _call_noalloc(lib, _lib, pool, batch, got, sgot, stream) == _lib.OK, lib.bikv_last_error()
        pool.check()                                                   # synchronises the stream, reads the status
        assert torch.equal(got, want) and torch.equal(sgot, swant), [len(r) for r in reqs]
        # and both equal the oracle's image
        assert got.numpy().tobytes() == oracle.gather_layered_c(pool_h, reqs, layout).tobytes()
        assert sgot.numpy().tobytes() == oracle.gather_layered_c(scale_h, reqs, layout).tobytes()
    stager.close()


def test_noalloc_gather_limits_and_errors(lib, cuda):
    import bikv_pagecopy as bk
    from bikv_pagecopy import _lib
    print("[case] allocation-free gather to host, limits", flush=True)
    # a tile larger than the scratch is refused with a clear message, nothing is enqueued
    big_d = torch.zeros((1, 2, (16 << 20) + 4096), dtype=torch.uint8, device=cuda)
    big = bk.PagedKVPool.from_stacked(big_d, plane_dims=1)
    b = big.make_batch([[1]])
    host = bk.pinned_empty(b.n_slots * big.tile_bytes).fill_(7)
    torch.cuda.synchronize(cuda)
    assert _call_noalloc(lib, _lib, big, b, host) == _lib.ERANGE
    assert b"exceeds the 16777216-byte scratch" in lib.bikv_last_error()
    assert bool((host == 7).all())
    # the usual argument checks
    small_d = torch.arange(2 * 8 * 4096, dtype=torch.int32, device=cuda).view(torch.uint8).view(2, 8, 4 * 4096)
    small = bk.PagedKVPool.from_stacked(small_d, plane_dims=1)
    sb = small.make_batch([[5, 2, 5]])
    short = bk.pinned_empty(4096)
    torch.cuda.synchronize(cuda)
    assert _call_noalloc(lib, _lib, small, sb, short) == _lib.ERANGE
    # the Python wrapper, with a rejected page id reported through the shared status word
    host = bk.pinned_empty(sb.n_slots * small.tile_bytes).fill_(0)
    bk.gather_to_host_noalloc(small, sb, host)
    small.check()
    assert torch.equal(host.view(2, 3, -1), small_d[:, [5, 2, 5]].cpu())
    sb.index[0, 1] = 99
    bk.gather_to_host_noalloc(small, sb, host)
    with pytest.raises(RuntimeError, match="page-id"):
        small.check()
    # an empty batch is a no-op
    eb = small.make_batch([[]])
    assert _call_noalloc(lib, _lib, small, eb, host) == _lib.OK


def test_noalloc_gather_allocates_nothing_and_replays_from_a_hip_graph(lib, oracle, cuda):
    """The two claims of the entry point's contract. (1) Device memory in use is the same before and after
    a call. (2) A call made while a stream is capturing records kernel nodes only, and the captured graph
    can be replayed: three replays, with the pool changed by eager work (and the host image cleared) between
    them, each checked against the oracle for the pool as it is at that moment."""
    import bikv_pagecopy as bk
    from bikv_pagecopy import _lib
    print("[case] allocation-free gather to host: memory use and graph replay", flush=True)
    assert lib.bikv_init(0) == _lib.OK
    rng = np.random.default_rng(73)
    n_planes, n_pages, tile = 4, 30, 1280 * 1024
    pool_h = rng.integers(0, 256, size=(n_planes, n_pages, tile), dtype=np.uint8)
    pool_d = torch.from_numpy(pool_h).to(cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    reqs = [rng.permutation(n_pages)[:9], rng.permutation(n_pages)[:4]]
    batch = pool.make_batch(reqs)
    host = bk.pinned_empty(batch.n_slots * tile)
    torch.cuda.synchronize(cuda)
    # (1) no allocation: free device memory as the driver reports it, before and after an eager call
    free_before = torch.cuda.mem_get_info(cuda)[0]
    stream = C.c_void_p(torch.cuda.current_stream(cuda).cuda_stream)
    assert _call_noalloc(lib, _lib, pool, batch, host, None, stream) == _lib.OK, lib.bikv_last_error()
    pool.check()
    assert torch.cuda.mem_get_info(cuda)[0] == free_before
    assert host.numpy().tobytes() == oracle.gather_layered_c(pool_h, reqs).tobytes()
    # (2) capture once, replay three times
    side = torch.cuda.Stream(device=cuda)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            s = C.c_void_p(torch.cuda.current_stream(cuda).cuda_stream)
            assert _call_noalloc(lib, _lib, pool, batch, host, None, s) == _lib.OK, lib.bikv_last_error()
    for rep in range(3):
        # eager work between replays: new bytes in some of the gathered pages, host image cleared
        page = int(reqs[0][rep])
        fresh = rng.integers(0, 256, size=(n_planes, tile), dtype=np.uint8)
        pool_h[:, page] = fresh
        pool_d[:, page] = torch.from_numpy(fresh).to(cuda)
        host.fill_(0xA5)
        torch.cuda.synchronize(cuda)
        graph.replay()
        torch.cuda.synchronize(cuda)
        assert host.numpy().tobytes() == oracle.gather_layered_c(pool_h, reqs).tobytes(), rep
    pool.check()
    del graph
    pool.close()
