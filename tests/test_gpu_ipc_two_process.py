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
