"""Device -> pinned-host staging on a real GPU: both modes against the oracle's staging image."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
@pytest.mark.parametrize("mode", ["pipelined", "direct"])
def test_gather_to_host_matches_oracle(lib, oracle, cuda, layout, mode):
    import bikv_pagecopy as bk
    print(f"[case] gather_to_host {layout} {mode}", flush=True)
    rng = np.random.default_rng(41)
    n_planes, n_pages, tile = 6, 90, 16384
    pool_h = rng.integers(0, 256, size=(n_planes, n_pages, tile), dtype=np.uint8)
    pool_d = torch.from_numpy(pool_h).to(cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    # request sizes around the chunk size: whole-plane-row chunks, split rows, a single page, empty
    reqs = [rng.permutation(n_pages)[:m] for m in (3, 40, 1, 0, 17)]
    batch = pool.make_batch(reqs, layout)
    want = oracle.gather_layered_c(pool_h, reqs, layout).tobytes()
    for chunk_tiles, n_buf in ((8, 2), (1, 3), (64, 1)):
        stager = bk.HostStager(cuda, chunk_bytes=chunk_tiles * tile, n_buffers=n_buf)
        host = bk.pinned_empty(batch.n_slots * tile)
        host.fill_(0xA5)
        nbytes, n_chunks, sec = stager.gather_to_host(pool, batch, host, mode)
        assert nbytes == batch.n_slots * tile and sec > 0
        assert host.numpy().tobytes() == want, (chunk_tiles, n_buf)
        if mode == "pipelined":
            plan = bk.plan_chunks(batch.req_pages, n_planes, layout, chunk_tiles)
            assert n_chunks == len(plan)
        stager.close()


@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
@pytest.mark.parametrize("mode", ["pipelined", "direct"])
def test_gather_to_host_moves_scales_with_the_payload(lib, oracle, cuda, layout, mode):
    """fp8-style pool: 16 KiB payload tiles + 32-byte scale tiles go to two pinned images."""
    import bikv_pagecopy as bk
    print(f"[case] gather_to_host with scales {layout} {mode}", flush=True)
    rng = np.random.default_rng(43)
    n_planes, n_pages, tile, stile = 10, 60, 16384, 32
    pool_h = rng.integers(0, 256, size=(n_planes, n_pages, tile), dtype=np.uint8)
    scale_h = rng.integers(0, 256, size=(n_planes, n_pages, stile), dtype=np.uint8)
    pool = bk.PagedKVPool.from_stacked(torch.from_numpy(pool_h).to(cuda), plane_dims=1,
                                       scale=torch.from_numpy(scale_h).to(cuda))
    reqs = [rng.permutation(n_pages)[:m] for m in (5, 31, 1, 0, 12)]
    batch = pool.make_batch(reqs, layout)
    want = oracle.gather_layered_c(pool_h, reqs, layout).tobytes()
    swant = oracle.gather_layered_c(scale_h, reqs, layout).tobytes()
    for chunk_tiles in (4, 1, 64):
        stager = bk.HostStager(cuda, chunk_bytes=chunk_tiles * tile, n_buffers=2)
        host = bk.pinned_empty(batch.n_slots * tile).fill_(0xA5)
        shost = bk.pinned_empty(batch.n_slots * stile).fill_(0xA5)
        nbytes, _, _ = stager.gather_to_host(pool, batch, host, mode, host_scale=shost)
        assert nbytes == batch.n_slots * (tile + stile)
        assert host.numpy().tobytes() == want and shost.numpy().tobytes() == swant, chunk_tiles
        stager.close()
    with pytest.raises(RuntimeError, match="host_scale"):
        bk.HostStager(cuda).gather_to_host(pool, batch, bk.pinned_empty(batch.n_slots * tile), mode)


def test_gather_to_host_argument_checks(lib, cuda):
    import bikv_pagecopy as bk
    print("[case] gather_to_host checks", flush=True)
    pool_d = torch.zeros((2, 8, 4096), dtype=torch.uint8, device=cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    batch = pool.make_batch([[1, 2, 3]])
    stager = bk.HostStager(cuda, chunk_bytes=4096, n_buffers=2)
    with pytest.raises(RuntimeError, match="pinned"):
        stager.gather_to_host(pool, batch, torch.empty(batch.n_slots * 4096, dtype=torch.uint8))
    with pytest.raises(RuntimeError, match="staging image needs"):
        stager.gather_to_host(pool, batch, bk.pinned_empty(4096))
    tiny = bk.HostStager(cuda, chunk_bytes=4096, n_buffers=1)
    big_d = torch.zeros((1, 4, 8192), dtype=torch.uint8, device=cuda)
    big = bk.PagedKVPool.from_stacked(big_d, plane_dims=1)
    with pytest.raises(RuntimeError, match="smaller than one tile"):
        tiny.gather_to_host(big, big.make_batch([[0]]), bk.pinned_empty(8192))
    with pytest.raises(RuntimeError):
        bk.HostStager(cuda, chunk_bytes=16, n_buffers=2)


def test_measure_d2h_runs(lib, cuda):
    import bikv_pagecopy as bk
    print("[case] d2h yardstick", flush=True)
    dev = torch.arange(0, 1 << 22, dtype=torch.int32, device=cuda).view(torch.uint8)
    host = bk.pinned_empty(dev.numel())
    for chunk in (0, 1 << 20):
        host.zero_()
        sec = bk.measure_d2h(cuda, host, dev, chunk)
        assert sec > 0 and torch.equal(host, dev.cpu())


@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
@pytest.mark.parametrize("mode", ["pipelined", "direct"])
def test_scatter_from_host_matches_oracle(lib, oracle, cuda, layout, mode):
    """Pinned staging image -> pool pages, payload and scales, at chunk sizes around the requests."""
    import bikv_pagecopy as bk
    print(f"[case] scatter_from_host {layout} {mode}", flush=True)
    rng = np.random.default_rng(47)
    n_planes, n_pages, tile, stile = 6, 90, 16384, 32
    pool_h = rng.integers(0, 256, size=(n_planes, n_pages, tile), dtype=np.uint8)
    scale_h = rng.integers(0, 256, size=(n_planes, n_pages, stile), dtype=np.uint8)
    perm = rng.permutation(n_pages)
    cuts = np.cumsum([3, 40, 1, 0, 17])
    reqs = [np.ascontiguousarray(a) for a in np.split(perm[:cuts[-1]], cuts[:-1])]
    n_slots = int(cuts[-1]) * n_planes
    image = rng.integers(0, 256, size=n_slots * tile, dtype=np.uint8)
    simage = rng.integers(0, 256, size=n_slots * stile, dtype=np.uint8)
    want = pool_h.copy()
    oracle.scatter_layered_c(want, reqs, image, layout)
    swant = scale_h.copy()
    oracle.scatter_layered_c(swant, reqs, simage, layout)
    for chunk_tiles, n_buf in ((8, 2), (1, 3), (64, 1)):
        pool_d = torch.from_numpy(pool_h).to(cuda)
        scale_d = torch.from_numpy(scale_h).to(cuda)
        pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1, scale=scale_d)
        batch = pool.make_batch(reqs, layout)
        stager = bk.HostStager(cuda, chunk_bytes=chunk_tiles * tile, n_buffers=n_buf)
        host = bk.pinned_empty(n_slots * tile)
        host.copy_(torch.from_numpy(image))
        shost = bk.pinned_empty(n_slots * stile)
        shost.copy_(torch.from_numpy(simage))
        nbytes, n_chunks, sec = stager.scatter_from_host(pool, batch, host, mode, host_scale=shost)
        assert nbytes == n_slots * (tile + stile) and sec > 0
        assert np.array_equal(pool_d.cpu().numpy(), want), (chunk_tiles, n_buf)
        assert np.array_equal(scale_d.cpu().numpy(), swant), (chunk_tiles, n_buf)
        # and back: the gather of the same pages returns the image
        back = bk.pinned_empty(n_slots * tile).fill_(0xA5)
        sback = bk.pinned_empty(n_slots * stile).fill_(0xA5)
        stager.gather_to_host(pool, batch, back, mode, host_scale=sback)
        assert back.numpy().tobytes() == image.tobytes() and sback.numpy().tobytes() == simage.tobytes()
        stager.close()
        pool.close()


def test_scatter_from_host_argument_checks(lib, cuda):
    import bikv_pagecopy as bk
    print("[case] scatter_from_host checks", flush=True)
    pool_d = torch.zeros((2, 8, 4096), dtype=torch.uint8, device=cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    batch = pool.make_batch([[1, 2, 3]])
    stager = bk.HostStager(cuda, chunk_bytes=4096, n_buffers=2)
    with pytest.raises(RuntimeError, match="pinned"):
        stager.scatter_from_host(pool, batch, torch.empty(batch.n_slots * 4096, dtype=torch.uint8))
    with pytest.raises(RuntimeError, match="staging image needs"):
        stager.scatter_from_host(pool, batch, bk.pinned_empty(4096))
    # an out-of-range page id is skipped and reported, the other pages land
    bad = pool.make_batch([[1, 2, 3]])
    bad.index[0, 1] = 99
    host = bk.pinned_empty(batch.n_slots * 4096).fill_(7)
    with pytest.raises(RuntimeError, match="page-id"):
        stager.scatter_from_host(pool, bad, host)
    got = pool_d.cpu()
    assert bool((got[:, 1] == 7).all()) and bool((got[:, 3] == 7).all()) and bool((got[:, 2] == 0).all())


def test_measure_h2d_runs(lib, cuda):
    import bikv_pagecopy as bk
    print("[case] h2d yardstick", flush=True)
    host = bk.pinned_empty(1 << 24)
    host.copy_(torch.arange(0, 1 << 22, dtype=torch.int32).view(torch.uint8))
    dev = torch.zeros(1 << 24, dtype=torch.uint8, device=cuda)
    for chunk in (0, 1 << 20):
        dev.zero_()
        sec = bk.measure_h2d(cuda, dev, host, chunk)
        assert sec > 0 and torch.equal(dev.cpu(), host)
