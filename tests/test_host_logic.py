"""Host-side logic and the C-ABI surface, without a GPU: index/offset builders against the oracle's
loop restatements, the staging chunk planner's invariants, workload generators, and that the shared
library loads, exports every symbol the header declares and rejects bad arguments loudly."""
import ctypes as C
import os
import re
import subprocess
import tempfile

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "bikv_pagecopy.h")


# ---- C ABI --------------------------------------------------------------------------------------
def test_library_exports_every_declared_symbol(lib):
    from bikv_pagecopy import _lib
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = set(re.findall(r"\b(bikv_[a-z0-9_]+)\s*\(", text))
    assert declared, "no declarations parsed"
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    assert declared == set(_lib.EXPORTED_SYMBOLS), "binding and header disagree"
    assert lib.bikv_abi_version() == _lib.ABI_VERSION


def test_shared_control_is_byte_compatible_with_the_reference():
    """ipc_wrapper.h:14-28 on x86-64 glibc: sizeof 480 and these offsets."""
    from bikv_pagecopy._lib import SharedControl
    want = {"sem_start": 0, "sem_complete": 32, "dtype_code": 64, "error_code": 68, "device_id": 72,
            "hostname": 76, "data_size": 336, "tensor_dim": 344, "current_offset": 352,
            "last_valid_offset": 360, "buffer_size": 368, "ipc_handle": 376, "tensor_shape": 440}
    assert C.sizeof(SharedControl) == 480
    for k, v in want.items():
        assert getattr(SharedControl, k).offset == v, k


def test_header_compiles_as_c_and_cxx_and_matches_a_reference_shaped_struct():
    """Compiles the header as C and as C++ (where its static_asserts run), next to a struct written
    with the reference's field types (sem_t, int, char[256], size_t, ...), and compares layouts."""
    src = r'''
#include <semaphore.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include "bikv_pagecopy.h"
struct RefShaped { sem_t a; sem_t b; int data_ready; int error_code; int device_id; char hostname[256];
  size_t data_size; size_t tensor_dim; size_t current_offset; size_t last_valid_offset; size_t buffer_size;
  unsigned char cuda_handle[64]; int64_t tensor_shape[5]; };
int main(void) {
  if (sizeof(struct RefShaped) != sizeof(bikv_shared_control)) return 1;
  if (offsetof(struct RefShaped, hostname) != offsetof(bikv_shared_control, hostname)) return 2;
  if (offsetof(struct RefShaped, cuda_handle) != offsetof(bikv_shared_control, ipc_handle)) return 3;
  if (offsetof(struct RefShaped, tensor_shape) != offsetof(bikv_shared_control, tensor_shape)) return 4;
  if (sizeof(bikv_tensor_dims) != 40) return 5;
  printf("%zu\n", sizeof(bikv_shared_control));
  return 0;
}
'''
    with tempfile.TemporaryDirectory() as td:
        for comp, ext in (("gcc", "c"), ("g++", "cpp")):
            p = os.path.join(td, f"t.{ext}")
            open(p, "w").write(src)
            exe = os.path.join(td, f"t_{ext}")
            subprocess.run([comp, "-I", os.path.join(ROOT, "include"), p, "-o", exe, "-lpthread"], check=True)
            out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout.strip()
            assert out == "480"


def test_bad_arguments_are_rejected_before_any_gpu_work(lib):
    from bikv_pagecopy import _lib
    assert lib.bikv_copy_runs(None, 0, None, 0, None, None, -1, 16, 1, None) == _lib.EINVAL
    assert "negative" in _lib.last_error()
    assert lib.bikv_copy_runs(None, 0, None, 0, None, None, 0, 16, 1, None) == _lib.OK  # empty batch
    assert lib.bikv_copy_runs(None, 64, None, 64, None, None, 4, 16, 1, None) == _lib.EINVAL
    buf = (C.c_ubyte * 64)()
    off = (C.c_int64 * 4)()
    p, o = C.addressof(buf), C.addressof(off)
    assert lib.bikv_copy_runs(p, 64, p, 64, o, o, 4, 16, 0, None) == _lib.EINVAL       # unit_bytes
    assert lib.bikv_copy_runs(p, 8, p, 64, o, o, 4, 16, 1, None) == _lib.EINVAL        # run > buffer
    d = _lib.PoolDesc()
    h = C.c_void_p()
    assert lib.bikv_pool_create(C.byref(d), C.byref(h)) == _lib.EINVAL and not h.value
    d.n_planes, d.n_pages, d.tile_bytes, d.page_stride_bytes = 2, 8, 64, 32
    assert lib.bikv_pool_create(C.byref(d), C.byref(h)) == _lib.EINVAL                 # stride < tile
    assert lib.bikv_set_tuning(b"unroll", 3) == _lib.EINVAL
    assert lib.bikv_set_tuning(b"no_such_knob", 1) == _lib.EINVAL
    assert lib.bikv_set_tuning(b"unroll", 4) == _lib.OK
    with pytest.raises(RuntimeError, match="unroll"):
        _lib.check(lib.bikv_set_tuning(b"unroll", 5))


def test_ring_roles_fail_loudly_when_uninitialised_or_misused(lib):
    """The reference throws std::runtime_error from its init paths (ipc_service.cpp:30,82,94-98)."""
    import ipc_service
    from bikv_pagecopy import _lib
    ipc_service.producer_cleanup()
    ipc_service.consumer_cleanup()  # idempotent, as in the reference
    with pytest.raises(RuntimeError, match="shm_open failed"):
        ipc_service.producer_init(0, "/bikv_test_no_such_object")
    dims = _lib.TensorDimsC(0, 128, 2, 28, 2)
    assert lib.bikv_producer_copy_pages(None, 0, None, None, 0, 16, C.byref(dims), 2, 0, None) == _lib.ESTATE
    assert lib.bikv_consumer_receive(0, None, None, None, None, None, None) == _lib.ESTATE
    with pytest.raises(RuntimeError):
        ipc_service.cuda_producer_copy_pages(None, None, None, None, None, 16, None)


def test_producer_init_rejects_a_control_block_from_another_host(lib):
    """Same-host check of ipc_service.cpp:91-98, forced from the host with a hand-made control block."""
    import ipc_service
    from bikv_pagecopy._lib import SharedControl
    name = f"/bikv_test_foreign_{os.getpid()}"
    path = "/dev/shm" + name
    ctrl = SharedControl()
    ctrl.hostname = b"some-other-machine"
    try:
        with open(path, "wb") as f:
            f.write(bytes(ctrl))
        with pytest.raises(RuntimeError, match="same host"):
            ipc_service.producer_init(0, name.encode())
        with open(path, "wb") as f:
            f.write(bytes(SharedControl()))  # created but not filled in yet: no ring to attach to
        with pytest.raises(RuntimeError, match="describes no ring yet"):
            ipc_service.producer_init(0, name)
        with open(path, "wb") as f:
            f.write(b"\0" * 100)  # too small to be a control block
        with pytest.raises(RuntimeError, match="smaller than the control block"):
            ipc_service.producer_init(0, name)
    finally:
        os.unlink(path)


def test_python_layer_has_no_cpu_fallback():
    """The product must not import the oracle, and a CPU pool is refused."""
    import torch
    import bikv_pagecopy as bk
    pkg = os.path.join(ROOT, "bi-kv_amd")
    for dirpath, _, files in os.walk(pkg):
        for fn in files:
            if fn.endswith((".py", ".hip", ".h", ".cpp")):
                assert "oracle" not in open(os.path.join(dirpath, fn)).read().lower(), fn
    with pytest.raises(RuntimeError, match="CUDA"):
        bk.PagedKVPool.from_planes([torch.zeros(4, 8)])


# ---- index builder ------------------------------------------------------------------------------
@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
def test_build_index_slots_reproduce_the_oracle_layout(oracle, layout):
    """Applying (slot + q*stride) by hand must place tiles exactly where the oracle's gather does."""
    from bikv_pagecopy import build_index
    rng = np.random.default_rng(21)
    n_planes, n_pool, tile = 6, 50, 4
    pool = rng.integers(0, 255, size=(n_planes, n_pool, tile), dtype=np.uint8)
    reqs = [rng.permutation(n_pool)[:7], np.zeros(0, np.int64), np.array([5, 5, 9]), rng.permutation(n_pool)[:1]]
    idx, req_pages = build_index(reqs, n_planes, layout)
    assert req_pages.tolist() == [7, 0, 3, 1]
    out = np.zeros((11 * n_planes, tile), dtype=np.uint8)
    for i in range(idx.shape[1]):
        for q in range(n_planes):
            out[idx[1, i] + q * idx[2, i]] = pool[q, idx[0, i]]
    assert out.tobytes() == oracle.gather_layered_c(pool, reqs, layout).tobytes()
    # every slot is written exactly once
    slots = (idx[1][:, None] + np.arange(n_planes)[None, :] * idx[2][:, None]).reshape(-1)
    assert sorted(slots.tolist()) == list(range(11 * n_planes))


def test_build_index_empty():
    from bikv_pagecopy import build_index
    idx, rp = build_index([], 4, "layer_major")
    assert idx.shape == (3, 0) and rp.size == 0


# ---- offset builder (kvcache.py:161-196) ---------------------------------------------------------
def test_build_run_offsets_matches_reference_loops(oracle):
    from bikv_pagecopy import build_run_offsets
    rng = np.random.default_rng(4)
    for trial in range(200):
        page_size = int(rng.integers(1, 64))
        n_items = int(rng.integers(0, 8))
        tokens = rng.integers(1, 300, size=n_items)
        lists = [rng.integers(0, 10_000, size=-(-int(t) // page_size)).tolist() for t in tokens]
        pairs = [(k, int(t)) for k, t in enumerate(tokens)]
        so, do, total = oracle.build_offsets_loops(lists, pairs, page_size, 1)
        off, tot = build_run_offsets(lists, tokens, page_size, unit="tokens")
        assert off[0].tolist() == so and off[1].tolist() == do and tot == total
        ept = 14336
        so, do, _ = oracle.build_offsets_loops(lists, pairs, page_size, ept)
        off, _ = build_run_offsets(lists, tokens, page_size, elements_per_token=ept)
        assert off[0].tolist() == so and off[1].tolist() == do


def test_build_run_offsets_items_with_no_pages_and_errors():
    from bikv_pagecopy import build_run_offsets
    off, tot = build_run_offsets([[], [3, 1], []], [0, 20, 0], 16, 2)
    assert off.tolist() == [[96, 32], [0, 32]] and tot == 20
    with pytest.raises(ValueError):
        build_run_offsets([[1]], [1, 2], 16)
    with pytest.raises(ValueError):
        build_run_offsets([[1]], [1], 0)


# ---- chunk planner ------------------------------------------------------------------------------
@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
def test_plan_chunks_tiles_the_staging_image_exactly(lib, layout):
    from bikv_pagecopy import build_index, plan_chunks
    rng = np.random.default_rng(6)
    for trial in range(40):
        n_planes = int(rng.integers(1, 9))
        req_pages = rng.integers(0, 40, size=int(rng.integers(0, 7)))
        max_slots = int(rng.integers(1, 60))
        plan = plan_chunks(req_pages, n_planes, layout, max_slots)
        total_slots = int(req_pages.sum()) * n_planes
        idx, _ = build_index([np.zeros(m, np.int64) for m in req_pages], n_planes, layout)
        covered = np.zeros(total_slots, dtype=np.int64)
        at = 0
        for first_page, n_pages, q0, qc, first_slot, n_slots in plan.tolist():
            assert first_slot == at, "chunks must follow each other without gaps"
            assert n_slots == n_pages * qc
            assert 0 < n_slots <= max_slots
            # the rectangle (pages x planes) must land exactly inside [first_slot, first_slot+n_slots)
            i = np.arange(first_page, first_page + n_pages)
            q = np.arange(q0, q0 + qc)
            slots = (idx[1][i][:, None] + q[None, :] * idx[2][i][:, None]).reshape(-1)
            assert slots.min() == first_slot and slots.max() == first_slot + n_slots - 1
            covered[slots] += 1
            at += n_slots
        assert at == total_slots and np.all(covered == 1)


def test_plan_chunks_rejects_bad_arguments(lib):
    from bikv_pagecopy import plan_chunks
    with pytest.raises(RuntimeError):
        plan_chunks([1, -2], 4, "layer_major", 8)
    with pytest.raises(RuntimeError):
        plan_chunks([1], 4, "layer_major", 0)


# ---- workloads ----------------------------------------------------------------------------------
def test_shapes_match_the_published_byte_counts():
    from bikv_pagecopy.workloads import SHAPES
    want = {"tiny": (4096, 8192), "qwen2_1p5b": (8192, 458752), "qwen2_7b": (16384, 917504),
            "llama3_8b": (65536, 4194304), "llama3_70b_fp8": (16384, 2626560)}
    for name, (tile, page_all) in want.items():
        assert SHAPES[name].tile_bytes == tile and SHAPES[name].page_bytes == page_all
    assert SHAPES["llama3_70b_fp8"].scale_tile_bytes == 32
    assert SHAPES["qwen2_7b"].pool_bytes == 917504 * 131072


def test_workload_generators_have_the_stated_properties():
    from bikv_pagecopy import workloads as w
    t = w.named("tiny")
    assert len(t["gather"][0]) == 64 == len(set(t["gather"][0].tolist()))
    assert t["gather"][0].tolist() != t["scatter"][0].tolist()

    s2 = w.SHAPES["qwen2_1p5b"]
    u = w.named("qwen2_1p5b")
    allids = np.concatenate(u["gather"])
    assert len(u["gather"]) == 32 and len(set(allids.tolist())) == len(allids)
    assert all(512 // 16 <= len(r) <= 4096 // 16 for r in u["gather"])
    assert allids.min() >= 0 and allids.max() < s2.n_pages
    assert not np.all(np.diff(allids) > 0)  # out of order by construction

    m = w.named("qwen2_7b")
    g, s = np.concatenate(m["gather"]), np.concatenate(m["scatter"])
    assert len(m["gather"]) == 32 == len(m["scatter"])
    dup = 1 - len(set(g.tolist())) / len(g)
    assert 0.05 < dup < 0.12, dup                      # ~10 % duplicated reads
    assert len(set(s.tolist())) == len(s)              # scatter ids unique
    assert not set(s.tolist()) & set(g.tolist())       # and freshly allocated
    assert w.named("qwen2_7b")["gather"][3].tolist() == m["gather"][3].tolist()  # seeded

    ln = w.named("llama3_8b")
    sizes = np.array([len(r) for r in ln["gather"]])
    assert len(sizes) == 128 and sizes.min() >= 1 and sizes.max() <= 16384 // 32
    assert 40 <= np.median(sizes) <= 90                # median 2048 tokens = 64 pages

    z = w.named("llama3_70b_fp8")
    sizes = np.array([len(r) for r in z["gather"]])
    assert len(sizes) == 256 and sizes.min() == 1 and sizes.max() <= 2048
    assert (sizes == 1).sum() >= 5                     # many single-page requests
    sc = np.concatenate(z["scatter"]) if z["scatter"] else np.zeros(0)
    assert len(set(sc.tolist())) == len(sc)

    small = w.mixed_gather_scatter(w.SHAPES["qwen2_7b"].scaled(512), 8, 1024, 8192, seed=3)
    assert sum(len(r) for r in small["gather"]) + sum(len(r) for r in small["scatter"]) <= 512


def test_build_run_offsets_can_return_the_tokens_of_each_run():
    from bikv_pagecopy.offsets import build_run_offsets
    pages_list = [[7, 2, 39], [4], [], [30, 31, 0], [5, 6]]
    tokens = [40, 16, 0, 33, 17]
    off, total = build_run_offsets(pages_list, tokens, 16, unit="tokens", with_sizes=True)
    assert off.shape == (3, 9) and total == 106
    assert off[2].tolist() == [16, 16, 8, 16, 16, 16, 1, 16, 1]
    assert off[1].tolist() == np.concatenate([[0], np.cumsum(off[2])[:-1]]).tolist()
    assert off[0].tolist() == [p * 16 for p in (7, 2, 39, 4, 30, 31, 0, 5, 6)]
    off2, total2 = build_run_offsets(pages_list, tokens, 16, unit="tokens")
    assert total2 == total and np.array_equal(off2, off[:2])
    e, t0 = build_run_offsets([], [], 16, with_sizes=True)
    assert e.shape == (3, 0) and t0 == 0


def test_plain_c_client_compiles_against_the_header_alone():
    """The C client used by the GPU suite must build with gcc -std=c99 -pedantic from the public header
    (no HIP headers on the include path)."""
    import subprocess
    import tempfile
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with tempfile.TemporaryDirectory() as tmp:
        r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(root, "include"),
                            "-c", os.path.join(root, "tests", "c_client", "abi_client.c"), "-o", os.path.join(tmp, "c.o")],
                           capture_output=True, text=True)
        assert r.returncode == 0, r.stderr


def test_producer_refuses_to_map_a_ring_of_2_gib_from_another_process(lib):
    """The check happens on the control block, before any GPU call: a control block that announces a
    2 GiB ring (written here by hand, as a consumer in another process would) is refused."""
    import mmap
    from bikv_pagecopy import _lib
    name = f"/bikv_test_bigring_{os.getpid()}"
    path = "/dev/shm" + name
    ctrl = _lib.SharedControl()
    host = os.uname().nodename.encode()
    ctrl.hostname = host
    ctrl.buffer_size = 2 << 30
    with open(path, "wb") as f:
        f.write(bytes(ctrl))
    try:
        rc = lib.bikv_producer_init(0, name.encode())
        assert rc == -6 and b"2 GiB" in lib.bikv_last_error()
        assert not lib.bikv_producer_control()
    finally:
        os.unlink(path)


def test_find_duplicate_names_the_first_repeated_destination(lib):
    """Host-side check for scatters (duplicate destinations race on the device, as they do in the
    reference's kernel, copy_kernel.cu:29-35), against a brute-force statement."""
    import numpy as np
    import bikv_pagecopy as bk
    from bikv_pagecopy import _lib
    bk.require_unique([])
    bk.require_unique([5])
    bk.require_unique(np.random.default_rng(0).permutation(1000))
    with pytest.raises(RuntimeError, match=r"id 7 is named more than once \(entries 1 and 4\)"):
        bk.require_unique([3, 7, 9, 2, 7, 3])
    with pytest.raises(RuntimeError, match=r"id -2 is named more than once \(entries 0 and 1\)"):
        bk.require_unique([-2, -2])
    rng = np.random.default_rng(1)
    for _ in range(200):
        ids = rng.integers(0, 40, size=rng.integers(0, 30)).astype(np.int64)
        seen, want = {}, None
        for i, v in enumerate(ids.tolist()):
            if v in seen:
                want = (v, seen[v], i)
                break
            seen.setdefault(v, i)
        dup = C.c_int64(-1)
        rc = lib.bikv_find_duplicate(ids.ctypes.data_as(C.POINTER(C.c_int64)), len(ids), C.byref(dup))
        if want is None:
            assert rc == _lib.OK
        else:
            assert rc == _lib.EINVAL and dup.value == want[0]
            assert f"(entries {want[1]} and {want[2]})".encode() in lib.bikv_last_error()
    assert lib.bikv_find_duplicate(None, 3, None) == _lib.EINVAL


def test_make_batch_can_refuse_duplicate_scatter_destinations():
    """build_index is pure host logic; the check sits in front of it in PagedKVPool.make_batch."""
    import numpy as np
    import bikv_pagecopy as bk
    from bikv_pagecopy.pool import build_index
    idx, _ = build_index([np.array([4, 9]), np.array([1, 9, 3])], 2, "layer_major")
    with pytest.raises(RuntimeError, match="scatter batch: destination id 9"):
        bk.require_unique(idx[0], "scatter batch")


def test_stage_times_report_has_the_reference_stages():
    from bikv_pagecopy import kvcache_calls as k
    t = k.StageTimes(pages=3, tokens=40, data_bytes=1 << 20, index_ms=0.1, upload_ms=0.2, copy_ms=0.5, total_ms=1.0)
    assert t.copy_MBps == pytest.approx(2000.0)
    text = t.report()
    for word in ("offset tables", "upload", "IPC page copy", "2000.00 MB/s", "total: 1.00 ms", "0.0250 ms per token"):
        assert word in text
