"""`ipc_service` with the producer and the consumer in two processes sharing one GPU, as the
reference's own scripts run it (Bi-KV/SharedMemory/CUDA_Shared/test_page_ipc.py:171-199): the consumer
creates the control block and the device ring and publishes the ring's IPC handle, the producer maps it
and copies pages into it, the consumer reads them through a non-owning view. Seeded data, shuffled
offsets, several transfers including ring wraps. The ring holds two and a half transfers (IPC mappings
are kept far below 2 GiB)."""
import multiprocessing as mp
import os
import sys
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PAGE_SIZE, DIMS, POOL_PAGES, N_RUNS, TRANSFERS = 8, (64, 2, 3, 2), 40, 23, 5
PAGE_ELEMS = PAGE_SIZE * DIMS[0] * DIMS[1] * DIMS[2] * DIMS[3]
PER_TRANSFER = N_RUNS * PAGE_ELEMS * 2
RING_BYTES = 5 * PER_TRANSFER // 2


def _paths():
    for p in (ROOT, os.path.join(ROOT, "bi-kv_amd")):
        if p not in sys.path:
            sys.path.insert(0, p)


def _transfer(k):
    rng = np.random.default_rng(1000 + k)
    ids = rng.integers(0, POOL_PAGES, size=N_RUNS)
    return ids * PAGE_ELEMS, rng.permutation(N_RUNS).astype(np.int64) * PAGE_ELEMS


def _pool():
    return np.random.default_rng(99).integers(0, 65536, size=POOL_PAGES * PAGE_ELEMS, dtype=np.uint16)


def _consumer(name, ready, go, out, backpressure=False):
    try:
        _paths()
        import torch
        import ipc_service
        ipc_service.consumer_init(0, name, RING_BYTES)
        ready.set()
        digests = []
        for k in range(TRANSFERS):
            t = ipc_service.consumer_receive(timeout_ms=60000)
            assert tuple(t.shape) == (N_RUNS * PAGE_SIZE,) + DIMS and t.dtype == torch.float16
            if backpressure:
                time.sleep(0.05)          # a slow consumer: the producer has time to run ahead
            digests.append(t.cpu().contiguous().view(torch.int16).numpy().tobytes())
            if backpressure:
                ipc_service.consumer_release()
            else:
                go.set()                  # the producer may overwrite the ring from here on
        ipc_service.consumer_cleanup()
        out.put(("consumer", "ok", digests))
    except Exception as e:  # noqa: BLE001
        out.put(("consumer", f"{type(e).__name__}: {e}", None))
        go.set()


def _producer(name, ready, go, out, backpressure=False):
    try:
        _paths()
        import torch
        import ipc_service
        if not ready.wait(120):
            raise RuntimeError("consumer did not come up")
        ipc_service.producer_init(0, name.encode())
        if backpressure:
            ipc_service.producer_set_backpressure(True, timeout_ms=60000)
        pool = torch.from_numpy(_pool().view(np.int16)).cuda().view(torch.float16)
        d = ipc_service.TensorDims()
        d.head_size, d.num_kv_heads, d.num_layers, d.kv_pair = DIMS
        for k in range(TRANSFERS):
            so, do = _transfer(k)
            ipc_service.producer_copy_pages(pool, torch.from_numpy(so).cuda(), torch.from_numpy(do).cuda(),
                                            PAGE_SIZE, d)
            if backpressure:
                continue                  # no handshake outside the ring: sem_complete paces the producer
            if not go.wait(120):
                raise RuntimeError("consumer did not acknowledge")
            go.clear()
        ipc_service.producer_cleanup()
        out.put(("producer", "ok", None))
    except Exception as e:  # noqa: BLE001
        out.put(("producer", f"{type(e).__name__}: {e}", None))


@pytest.mark.parametrize("backpressure", [False, True])
def test_two_process_page_copy_over_hip_ipc(oracle, cuda, backpressure):
    """backpressure=False: the reference's protocol, paced by an event outside the ring (its scripts
    sleep instead). backpressure=True: a free-running producer and a slow consumer, paced only by
    sem_complete."""
    print(f"[case] ipc_service two processes, backpressure={backpressure}", flush=True)
    ctx = mp.get_context("spawn")
    name = f"/bikv_test_2proc_{os.getpid()}_{int(backpressure)}"
    ready, go, out = ctx.Event(), ctx.Event(), ctx.Queue()
    procs = [ctx.Process(target=_consumer, args=(name, ready, go, out, backpressure)),
             ctx.Process(target=_producer, args=(name, ready, go, out, backpressure))]
    for p in procs:
        p.start()
    results = {}
    try:
        for _ in procs:
            who, status, payload = out.get(timeout=240)
            results[who] = (status, payload)
    finally:
        for p in procs:
            p.join(timeout=30)
            if p.is_alive():
                p.terminate()
        try:
            os.unlink("/dev/shm" + name)
        except FileNotFoundError:
            pass
    assert results["producer"][0] == "ok", results
    assert results["consumer"][0] == "ok", results
    pool = _pool()
    assert 2 * PER_TRANSFER <= RING_BYTES < TRANSFERS * PER_TRANSFER, "the sequence must wrap the ring"
    for k, got in enumerate(results["consumer"][1]):
        so, do = _transfer(k)
        want = np.zeros(N_RUNS * PAGE_ELEMS, dtype=np.uint16)
        oracle.copy_runs_c(pool, want, so, do, PAGE_ELEMS)
        assert got == want.tobytes(), f"transfer {k} differs"


# ---- a whole transfer between two processes: layered gather -> ring -> layered scatter -------------
L_PLANES, L_PAGES, L_TILE, L_TRANSFERS = 4, 40, 8192, 4


def _layer_pool(seed):
    return np.random.default_rng(seed).integers(0, 256, size=(L_PLANES, L_PAGES, L_TILE), dtype=np.uint8)


def _layer_transfer(k):
    rng = np.random.default_rng(2000 + k)
    src = [rng.permutation(L_PAGES)[:7], rng.permutation(L_PAGES)[:5]]          # gathered from the sender's pool
    perm = rng.permutation(L_PAGES)
    dst = [perm[:7], perm[7:12]]                                                # unique pages of the receiver's pool
    return src, dst


def _layer_receiver(name, ready, out):
    try:
        _paths()
        import torch
        import ipc_service
        import bikv_pagecopy as bk
        per = 12 * L_PLANES * L_TILE
        ipc_service.consumer_init(0, name, 5 * per // 2)
        ready.set()
        pool_d = torch.from_numpy(_layer_pool(7)).cuda()
        pool = bk.PagedKVPool.from_stacked(pool_d, plane_dims=1)
        for k in range(L_TRANSFERS):
            _, dst = _layer_transfer(k)
            t = ipc_service.consumer_receive(timeout_ms=60000)
            assert tuple(t.shape) == (L_PLANES, 12, L_TILE) and t.dtype == torch.uint8
            pool.scatter(pool.make_batch(dst, "layer_major"), t.reshape(-1))
            pool.check()                                    # the ring window has been read
            ipc_service.consumer_release()
        digest = pool_d.cpu().numpy().tobytes()
        ipc_service.consumer_cleanup()
        out.put(("receiver", "ok", digest))
    except Exception as e:  # noqa: BLE001
        out.put(("receiver", f"{type(e).__name__}: {e}", None))


def _layer_sender(name, ready, out):
    try:
        _paths()
        import torch
        import ipc_service
        import bikv_pagecopy as bk
        if not ready.wait(120):
            raise RuntimeError("receiver did not come up")
        ipc_service.producer_init(0, name)
        ipc_service.producer_set_backpressure(True, timeout_ms=60000)
        pool = bk.PagedKVPool.from_stacked(torch.from_numpy(_layer_pool(5)).cuda(), plane_dims=1)
        for k in range(L_TRANSFERS):
            src, _ = _layer_transfer(k)
            batch = pool.make_batch(src, "layer_major")
            window = ipc_service.producer_reserve(batch.n_slots * L_TILE)
            pool.gather(batch, window)                      # kernels store into the receiver's memory
            ipc_service.producer_publish((L_PLANES, 12, L_TILE), torch.uint8)
        ipc_service.producer_cleanup()
        out.put(("sender", "ok", None))
    except Exception as e:  # noqa: BLE001
        out.put(("sender", f"{type(e).__name__}: {e}", None))


def test_two_process_layered_transfer(oracle, cuda):
    """Sender gathers request pages of its paged pool straight into the receiver's ring (the ring is
    the staging image, mapped through a HIP IPC handle); the receiver scatters each image into pages of
    its own pool. Paced by sem_complete only. The receiver's final pool must equal the oracle's."""
    print("[case] two processes: layered gather -> ring -> layered scatter", flush=True)
    ctx = mp.get_context("spawn")
    name = f"/bikv_test_2proc_layer_{os.getpid()}"
    ready, out = ctx.Event(), ctx.Queue()
    procs = [ctx.Process(target=_layer_receiver, args=(name, ready, out)),
             ctx.Process(target=_layer_sender, args=(name, ready, out))]
    for p in procs:
        p.start()
    results = {}
    try:
        for _ in procs:
            who, status, payload = out.get(timeout=240)
            results[who] = (status, payload)
    finally:
        for p in procs:
            p.join(timeout=30)
            if p.is_alive():
                p.terminate()
        try:
            os.unlink("/dev/shm" + name)
        except FileNotFoundError:
            pass
    assert results["sender"][0] == "ok", results
    assert results["receiver"][0] == "ok", (results["receiver"][0], results["sender"][0])
    src_pool, want = _layer_pool(5), _layer_pool(7)
    for k in range(L_TRANSFERS):
        src, dst = _layer_transfer(k)
        image = oracle.gather_layered_c(src_pool, src, "layer_major")
        oracle.scatter_layered_c(want, dst, image, "layer_major")
    assert results["receiver"][1] == want.tobytes()


def _placer(tag, start, out):
    """One tenant of the GPU: places an 8 GB pool through bikv_device_alloc, writes a page of it, gathers it."""
    try:
        _paths()
        import torch
        import bikv_pagecopy as bk
        torch.cuda.init()
        if not start.wait(120):
            raise RuntimeError("start signal did not come")
        t0 = time.time()
        buf = bk.DeviceBuffer(8 << 30, "cuda:0", spread=True, max_filler_bytes=16 << 30)
        wall = time.time() - t0
        n_planes, tile = 4, 16384
        n_pages = (8 << 30) // (n_planes * tile)
        pool_t = buf.tensor.view(n_planes, n_pages, tile)
        ids = np.array([0, n_pages // 2, n_pages - 1], dtype=np.int64)
        pool_t[:, torch.from_numpy(ids).cuda()] = tag
        pool = bk.PagedKVPool.from_stacked(pool_t, plane_dims=1)
        st, _ = pool.gather(pool.make_batch([ids]))
        pool.check()
        ok = bool((st == tag).all().item())
        pool.close()
        info = dict(buf.info)
        del pool_t, st
        buf.free()
        out.put((tag, "ok" if ok else "gathered bytes differ", info, wall))
    except Exception as e:  # noqa: BLE001
        out.put((tag, f"{type(e).__name__}: {e}", None, 0.0))


def test_two_processes_place_their_pools_on_one_gpu_at_the_same_time(cuda):
    """Bi-KV runs a cache process and a worker process per GPU. Two processes call bikv_device_alloc for 8 GB
    each at the same moment: the placements are serialised by the per-GPU file lock, both complete, both
    report their bookkeeping, and both pools move pages correctly."""
    print("[case] two processes place pools at once", flush=True)
    ctx = mp.get_context("spawn")
    start, out = ctx.Event(), ctx.Queue()
    procs = [ctx.Process(target=_placer, args=(tag, start, out)) for tag in (11, 22)]
    for p in procs:
        p.start()
    time.sleep(1.0)
    start.set()
    results = [out.get(timeout=300) for _ in procs]
    for p in procs:
        p.join(60)
        assert p.exitcode == 0
    for tag, status, info, wall in results:
        assert status == "ok", (tag, status)
        assert info["bytes"] >= 8 << 30 and info["n_chunks"] * info["chunk_bytes"] == info["bytes"]
        assert info["n_fillers"] * info["chunk_bytes"] <= 16 << 30
        assert info["seconds"] > 0 and wall >= info["seconds"] * 0.5
    print("   placements:", [(r[0], r[2]) for r in results], flush=True)
