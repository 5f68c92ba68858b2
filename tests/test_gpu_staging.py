"""Device -> pinned-host staging on a real GPU: both modes against the oracle's staging image."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
@pytest.mark.parametrize("mode", ["pipelined", "direct", "pipelined_kernel"])
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
    for chunk_tiles, n_buf, group in ((8, 2, 1), (1, 3, 1), (64, 1, 1), (2, 2, 4), (1, 2, 8), (3, 3, 2)):
        stager = bk.HostStager(cuda, chunk_bytes=chunk_tiles * tile, n_buffers=n_buf, chunks_per_launch=group)
        host = bk.pinned_empty(batch.n_slots * tile)
        host.fill_(0xA5)
        nbytes, n_chunks, sec = stager.gather_to_host(pool, batch, host, mode)
        assert nbytes == batch.n_slots * tile and sec > 0
        assert host.numpy().tobytes() == want, (chunk_tiles, n_buf, group)
        if mode == "pipelined":
            # one launch per piece of the plan, one host copy per chunk_bytes of a piece
            plan = bk.plan_chunks(batch.req_pages, n_planes, layout, chunk_tiles * group)
            assert n_chunks == sum(-(-int(p[5]) // chunk_tiles) for p in plan)
        elif mode == "pipelined_kernel":
            # one gather launch and one copy launch per piece of the plan
            assert n_chunks == len(bk.plan_chunks(batch.req_pages, n_planes, layout, chunk_tiles * group))
        else:
            assert n_chunks == 1
        stager.close()


@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
@pytest.mark.parametrize("mode", ["pipelined", "direct", "pipelined_kernel"])
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
    for chunk_tiles, group in ((4, 1), (1, 1), (64, 1), (2, 4)):
        stager = bk.HostStager(cuda, chunk_bytes=chunk_tiles * tile, n_buffers=2, chunks_per_launch=group)
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
    tiny = bk.HostStager(cuda, chunk_bytes=4096, n_buffers=1, chunks_per_launch=1)
    big_d = torch.zeros((1, 4, 8192), dtype=torch.uint8, device=cuda)
    big = bk.PagedKVPool.from_stacked(big_d, plane_dims=1)
    with pytest.raises(RuntimeError, match="smaller than one tile"):
        tiny.gather_to_host(big, big.make_batch([[0]]), bk.pinned_empty(8192), "pipelined")
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
@pytest.mark.parametrize("mode", ["pipelined", "direct", "pipelined_kernel"])
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
    for chunk_tiles, n_buf, group in ((8, 2, 1), (1, 3, 1), (64, 1, 1), (2, 2, 4)):
        pool_d = torch.from_numpy(pool_h).to(cuda)
        scale_d = torch.from_numpy(scale_h).to(cuda)
        pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1, scale=scale_d)
        batch = pool.make_batch(reqs, layout)
        stager = bk.HostStager(cuda, chunk_bytes=chunk_tiles * tile, n_buffers=n_buf, chunks_per_launch=group)
        host = bk.pinned_empty(n_slots * tile)
        host.copy_(torch.from_numpy(image))
        shost = bk.pinned_empty(n_slots * stile)
        shost.copy_(torch.from_numpy(simage))
        nbytes, n_chunks, sec = stager.scatter_from_host(pool, batch, host, mode, host_scale=shost)
        assert nbytes == n_slots * (tile + stile) and sec > 0
        assert np.array_equal(pool_d.cpu().numpy(), want), (chunk_tiles, n_buf, group)
        assert np.array_equal(scale_d.cpu().numpy(), swant), (chunk_tiles, n_buf, group)
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
        stager.scatter_from_host(pool, bad, host, "pipelined")
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


@pytest.mark.parametrize("mode", ["pipelined", "direct", "auto"])
def test_requests_enqueued_back_to_back_share_the_lanes(lib, oracle, cuda, mode):
    """Enqueue-only form: several requests go onto the lanes without a drain in between, each into its
    own part of the pinned region; one wait() completes them all. Then the same images travel back into
    other pages, also enqueued back to back."""
    import bikv_pagecopy as bk
    print(f"[case] asynchronous staging {mode}", flush=True)
    rng = np.random.default_rng(53)
    n_planes, n_pages, tile = 8, 120, 16384
    pool_h = rng.integers(0, 256, size=(n_planes, n_pages, tile), dtype=np.uint8)
    pool_d = torch.from_numpy(pool_h).to(cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    perm = rng.permutation(n_pages)
    sizes = [7, 1, 19, 4, 11]
    cuts = np.cumsum(sizes)
    reqs = [np.ascontiguousarray(a) for a in np.split(perm[:cuts[-1]], cuts[:-1])]
    stager = bk.HostStager(cuda, chunk_bytes=2 * tile, n_buffers=2, chunks_per_launch=2)
    images = [bk.pinned_empty(len(r) * n_planes * tile).fill_(0xA5) for r in reqs]
    batches = [pool.make_batch([r], "layer_major") for r in reqs]       # uploads queue on the current stream
    for b, img in zip(batches, images):
        stager.gather_to_host_async(pool, b, img, mode)
    nbytes, copies, sec = stager.wait()
    assert nbytes == sum(img.numel() for img in images) and copies >= len(reqs) and sec > 0
    for r, img in zip(reqs, images):
        assert img.numpy().tobytes() == oracle.gather_layered_c(pool_h, [r]).tobytes()
    # back into fresh pages
    fresh = perm[cuts[-1]: 2 * cuts[-1]]
    dst = [np.ascontiguousarray(a) for a in np.split(fresh, cuts[:-1])]
    want = pool_h.copy()
    for d, img in zip(dst, images):
        oracle.scatter_layered_c(want, [d], img.numpy())
    sbatches = [pool.make_batch([d], "layer_major") for d in dst]
    for b, img in zip(sbatches, images):
        stager.scatter_from_host_async(pool, b, img, mode)
    stager.wait()
    assert np.array_equal(pool_d.cpu().numpy(), want)
    # a rejected id in one of several enqueued requests is reported by the wait, the others land
    bad = pool.make_batch([dst[0]], "layer_major")
    bad.index[0, 0] = n_pages + 5
    stager.gather_to_host_async(pool, batches[1], images[1].fill_(0), mode)
    stager.gather_to_host_async(pool, bad, images[0], mode)
    with pytest.raises(RuntimeError, match="page-id"):
        stager.wait()
    assert images[1].numpy().tobytes() == oracle.gather_layered_c(pool_h, [reqs[1]]).tobytes()
    assert stager.wait()[0] == 0            # nothing pending, status cleared
    stager.close()


@pytest.mark.parametrize("chunk_mib,lanes,group", [(4, 2, 4), (8, 2, 4), (16, 2, 2), (4, 4, 1), (16, 4, 1)])
def test_llama3_8b_requests_staged_in_4_to_16_mib_chunks(lib, oracle, cuda, chunk_mib, lanes, group):
    """The Llama-3-8B-shaped workload itself: 64 KiB tiles x 64 planes (4 MiB per logical page), the
    leading requests of its log-normal stream, device -> pinned host in 4-16 MiB chunks and back, both
    modes, against the oracle's staging image."""
    import bikv_pagecopy as bk
    from bikv_pagecopy import workloads as w
    shape = w.SHAPES["llama3_8b"].scaled(160)                 # 160 pages x 4 MiB = 640 MiB pool
    print(f"[case] llama3_8b staging {chunk_mib} MiB x {lanes} lanes x {group} per launch", flush=True)
    assert shape.tile_bytes == 65536 and shape.n_planes == 64
    # the leading requests of the real stream (its length distribution, ids of this pool), each cut to at
    # most 30 pages = 120 MiB of staging image
    reqs = [r[:30] for r in w.named("llama3_8b", shape)["gather"][:5]]
    assert len(reqs) == 5 and len({len(r) for r in reqs}) > 1
    rng = np.random.default_rng(59)
    pool_h = rng.integers(0, 256, size=(shape.n_planes, shape.n_pages, shape.tile_bytes), dtype=np.uint8)
    pool_d = torch.from_numpy(pool_h).to(cuda)
    pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
    stager = bk.HostStager(cuda, chunk_bytes=chunk_mib << 20, n_buffers=lanes, chunks_per_launch=group)
    for mode in ("pipelined", "direct"):
        for r in reqs:
            b = pool.make_batch([r], "layer_major")
            host = bk.pinned_empty(b.n_slots * shape.tile_bytes).fill_(0xA5)
            stager.gather_to_host(pool, b, host, mode)
            want = oracle.gather_layered_c(pool_h, [r])
            assert host.numpy().tobytes() == want.tobytes(), (mode, len(r))
    # and the way back: the last image into the pages next to the ones it came from
    shifted = (np.asarray(reqs[-1]) + 1) % shape.n_pages
    sb = pool.make_batch([shifted], "layer_major", check_unique=True)
    stager.scatter_from_host(pool, sb, host, "pipelined")
    oracle.scatter_layered_c(pool_h, [shifted], host.numpy())
    assert np.array_equal(pool_d.cpu().numpy(), pool_h)
    stager.close()
    pool.close()


def test_a_rejected_page_id_is_reported_by_its_own_stager_only(lib, oracle, cuda):
    """Two stagers work on one pool at once; the batch given to the first names a page outside the pool.
    Only that stager's wait raises (every stager has status words of its own); the other's image equals the
    oracle's, and so do the good pages of the bad batch (the kernel skips the rejected page, nothing faults).
    Both orders of waiting, both sending modes."""
    import bikv_pagecopy as bk
    print("[case] per-stager status words", flush=True)
    rng = np.random.default_rng(401)
    n_planes, n_pages, tile = 4, 50, 4096
    pool_h = rng.integers(0, 256, size=(n_planes, n_pages, tile), dtype=np.uint8)
    pool = bk.PagedKVPool.from_stacked(torch.from_numpy(pool_h).to(cuda), plane_dims=1)
    good_req = [rng.permutation(n_pages)[:20]]
    bad_req = [np.array([3, n_pages + 5, 9, 11], dtype=np.int64)]
    good, bad = pool.make_batch(good_req), pool.make_batch(bad_req)
    want_good = oracle.gather_layered_c(pool_h, good_req).tobytes()
    want_bad = oracle.gather_layered_c(pool_h, [np.array([3, 9, 11])]).reshape(n_planes, 3, tile)
    for mode in ("direct", "pipelined", "pipelined_kernel"):
        for bad_waits_first in (True, False):
            a = bk.HostStager(cuda, chunk_bytes=4 * tile, n_buffers=2, chunks_per_launch=1)
            b = bk.HostStager(cuda, chunk_bytes=4 * tile, n_buffers=2, chunks_per_launch=1)
            host_a = bk.pinned_empty(bad.n_slots * tile).fill_(0xA5)
            host_b = bk.pinned_empty(good.n_slots * tile).fill_(0xA5)
            a.gather_to_host_async(pool, bad, host_a, mode)
            b.gather_to_host_async(pool, good, host_b, mode)
            if bad_waits_first:
                with pytest.raises(RuntimeError, match="page-id"):
                    a.wait()
                b.wait()
            else:
                b.wait()
                with pytest.raises(RuntimeError, match="page-id"):
                    a.wait()
            a.wait()                       # the report was consumed: a second wait is clean
            assert host_b.numpy().tobytes() == want_good, (mode, bad_waits_first)
            got = host_a.numpy().reshape(n_planes, 4, tile)
            assert np.array_equal(got[:, [0, 2, 3]], want_bad)
            if mode == "direct":           # the other modes copy whole lane buffers, skipped slots included
                assert (got[:, 1] == 0xA5).all()
            # neither report leaked into the words bikv_check_status reads
            pool.check()
            a.close()
            b.close()


def test_stager_banks_are_returned_when_a_stager_is_destroyed(lib, cuda):
    """A device hands out one set of status words per live stager; closing a stager gives its set back, so
    creating and closing many stagers one after the other never runs out."""
    import bikv_pagecopy as bk
    print("[case] stager banks recycled", flush=True)
    for _ in range(600):
        bk.HostStager(cuda, chunk_bytes=4096, n_buffers=1, chunks_per_launch=1).close()
    live = [bk.HostStager(cuda, chunk_bytes=4096, n_buffers=1, chunks_per_launch=1) for _ in range(8)]
    for s in live:
        s.close()


def test_stager_trace_records_every_step_of_a_transfer(lib, oracle, cuda):
    """The opt-in trace brackets every kernel launch and host copy with events: the steps it reports are those
    of the plan, in issue order, each with end >= start, and the transfer is still bit-exact."""
    import bikv_pagecopy as bk
    print("[case] stager trace", flush=True)
    rng = np.random.default_rng(409)
    n_planes, n_pages, tile = 6, 64, 16384
    pool_h = rng.integers(0, 256, size=(n_planes, n_pages, tile), dtype=np.uint8)
    pool = bk.PagedKVPool.from_stacked(torch.from_numpy(pool_h).to(cuda), plane_dims=1)
    reqs = [rng.permutation(n_pages)[:m] for m in (7, 30)]
    batch = pool.make_batch(reqs)
    want = oracle.gather_layered_c(pool_h, reqs).tobytes()
    stager = bk.HostStager(cuda, chunk_bytes=4 * tile, n_buffers=2, chunks_per_launch=2)
    plan = bk.plan_chunks(batch.req_pages, n_planes, "layer_major", 8)
    host = bk.pinned_empty(batch.n_slots * tile)
    for mode, copy_kind in (("pipelined", "copy_d2h"), ("pipelined_kernel", "copy_kernel")):
        stager.trace(4096)
        host.fill_(0xA5)
        stager.gather_to_host(pool, batch, host, mode)
        steps = stager.trace_read()
        assert host.numpy().tobytes() == want
        kernels = [s for s in steps if s["kind"] == "kernel"]
        copies = [s for s in steps if s["kind"] == copy_kind]
        assert len(kernels) == len(plan) and len(kernels) + len(copies) == len(steps)
        assert [s["bytes"] for s in kernels] == [int(p[5]) * tile for p in plan]
        assert sum(s["bytes"] for s in copies) == batch.n_slots * tile
        assert all(s["end_ms"] >= s["start_ms"] >= 0 for s in steps)
        assert {s["lane"] for s in steps} == {0, 1}
    # direct mode: one kernel step
    stager.trace(8)
    host.fill_(0)
    stager.gather_to_host(pool, batch, host, "direct")
    assert [s["kind"] for s in stager.trace_read()] == ["kernel"]
    assert host.numpy().tobytes() == want
    # a cap smaller than the transfer: the trace stops, the transfer does not
    stager.trace(3)
    host.fill_(0)
    stager.gather_to_host(pool, batch, host, "pipelined")
    assert len(stager.trace_read()) == 3
    assert host.numpy().tobytes() == want
    # the receiving direction (this changes the pool, hence last)
    stager.trace(64)
    perm = rng.permutation(n_pages)
    sb = pool.make_batch([perm[:9]], check_unique=True)
    stager.scatter_from_host(pool, sb, host[: sb.n_slots * tile], "pipelined")
    kinds = [s["kind"] for s in stager.trace_read()]
    assert kinds.count("copy_h2d") >= 1 and kinds.count("kernel") >= 1 and set(kinds) == {"copy_h2d", "kernel"}
    stager.trace(0)
    assert stager.trace_read() == []
    stager.close()
