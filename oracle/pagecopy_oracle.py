"""CPU oracle for the KV page-copy path — TEST INFRASTRUCTURE ONLY.

Nothing under bi-kv_amd/ may import this module: it is the checker, not a fallback. It is used by
tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py.

Three independent statements of the same semantics, so that they can be checked against each other:
  * `*_c`     — the C restatement in pagecopy_oracle.c, through ctypes;
  * `*_np`    — numpy fancy indexing on a [pages, tile] view (the library routine the formula
                reduces to);
  * `*_loops` — pure-Python per-byte / per-page loops that follow the reference line by line, for
                tiny inputs only.
plus `*_torch`, the reference's CPU path as a library routine (torch.index_select / index_copy_ on
host tensors; the vectorised form of the disabled host gather Bi-KV/Worker/Worker.py:207), which
the benchmark times as the CPU baseline.

Reference lines restated: Bi-KV/SharedMemory/CUDA_Shared/copy_kernel.cu:9-66 (the two kernels),
:81-89,116-127 (ring step), ipc_service.cpp:118-138 (producer_send bookkeeping),
Bi-KV/DistributedStorage/kvcache.py:161-174,187-196 (offset tables).
All functions are pinned by tests/test_oracle.py; none is "parity unpinned".
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle_pagecopy.so")
_clib = None


class Ring(C.Structure):
    _fields_ = [("data_size", C.c_uint64), ("tensor_dim", C.c_uint64), ("current_offset", C.c_uint64),
                ("last_valid_offset", C.c_uint64), ("buffer_size", C.c_uint64),
                ("tensor_shape", C.c_int64 * 5)]


def build():
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def clib():
    global _clib
    if _clib is None:
        if not os.path.exists(_SO):
            build()
        lib = C.CDLL(_SO)
        i64p, u8p = C.POINTER(C.c_int64), C.c_void_p
        lib.oracle_copy_runs.restype = C.c_int64
        lib.oracle_copy_runs.argtypes = [u8p, C.c_int64, u8p, C.c_int64, i64p, i64p, C.c_int64, C.c_int64, C.c_int64]
        lib.oracle_copy_runs_ragged.restype = C.c_int64
        lib.oracle_copy_runs_ragged.argtypes = [u8p, C.c_int64, u8p, C.c_int64, i64p, i64p, i64p, C.c_int64,
                                                C.c_int64, C.c_int64]
        lib.oracle_ring_step.restype = C.c_uint64
        lib.oracle_ring_step.argtypes = [C.POINTER(Ring)] + [C.c_int64] * 7
        lib.oracle_ring_send.restype = C.c_uint64
        lib.oracle_ring_send.argtypes = [C.POINTER(Ring), C.c_uint64, i64p, C.c_uint64]
        lib.oracle_build_offsets.restype = C.c_int64
        lib.oracle_build_offsets.argtypes = [i64p, i64p, i64p, C.c_int64, C.c_int64, C.c_int64, i64p, i64p]
        for name in ("oracle_gather_layered", "oracle_scatter_layered"):
            fn = getattr(lib, name)
            fn.restype = C.c_int64
            fn.argtypes = [C.POINTER(C.c_void_p), C.c_int32, C.c_int64, C.c_int64, C.c_int64, i64p, i64p,
                           C.c_int64, C.c_int32, u8p]
        lib.oracle_transpose_pages.restype = C.c_int64
        lib.oracle_transpose_pages.argtypes = [C.POINTER(C.c_void_p)] + [C.c_int32] * 5 + [C.c_int64] * 4 + \
            [u8p, C.c_int64, i64p, i64p, C.c_int64, C.c_int32]
        _clib = lib
    return _clib


def _i64(a):
    a = np.ascontiguousarray(a, dtype=np.int64)
    return a, a.ctypes.data_as(C.POINTER(C.c_int64))


def _bytes_view(a: np.ndarray) -> np.ndarray:
    assert a.flags.c_contiguous
    return a.reshape(-1).view(np.uint8)


# ---------------------------------------------------------------------------------------------
# run copy  (copy_kernel.cu:9-66)
# ---------------------------------------------------------------------------------------------
def copy_runs_c(src: np.ndarray, dst: np.ndarray, src_off, dst_off, run_elems: int) -> int:
    """In place on dst. Offsets and run length in elements of src/dst. Returns skipped runs."""
    es = src.dtype.itemsize
    assert dst.dtype.itemsize == es
    s, d = _bytes_view(src), _bytes_view(dst)
    so, sop = _i64(src_off)
    do, dop = _i64(dst_off)
    return clib().oracle_copy_runs(s.ctypes.data, s.size, d.ctypes.data, d.size, sop, dop, len(so),
                                   int(run_elems) * es, es)


def copy_runs_ragged_c(src: np.ndarray, dst: np.ndarray, src_off, dst_off, run_len, max_run_units: int,
                       unit_elems: int = 1) -> int:
    """In place on dst. Offsets and lengths in units of `unit_elems` elements. Returns skipped runs."""
    es = src.dtype.itemsize
    assert dst.dtype.itemsize == es
    s, d = _bytes_view(src), _bytes_view(dst)
    so, sop = _i64(src_off)
    do, dop = _i64(dst_off)
    ln, lnp = _i64(run_len)
    unit = int(unit_elems) * es
    return clib().oracle_copy_runs_ragged(s.ctypes.data, s.size, d.ctypes.data, d.size, sop, dop, lnp,
                                          len(so), int(max_run_units) * unit, unit)


def packed_items_np(pool_tokens: np.ndarray, cache_pages_list, item_tokens, page_size: int) -> np.ndarray:
    """What a packed transfer must deliver, stated without offsets: for every item, the rows of its
    pages in list order, cut to the item's token count, items back to back. pool_tokens is
    [n_pool_tokens, ...] (token-major pool, kvcache.py:38-43)."""
    parts = []
    for pages, tokens in zip(cache_pages_list, item_tokens):
        if len(pages) == 0:
            continue
        rows = np.concatenate([pool_tokens[p * page_size:(p + 1) * page_size] for p in pages])
        full = (len(pages) - 1) * page_size
        tail = tokens % page_size or page_size
        parts.append(rows[: full + tail])
    if not parts:
        return pool_tokens[:0]
    return np.concatenate(parts)


def copy_runs_np(src: np.ndarray, dst: np.ndarray, src_off, dst_off, run_elems: int):
    """numpy form: one fancy-index gather and one fancy-index assignment."""
    so = np.asarray(src_off, dtype=np.int64)[:, None] + np.arange(run_elems, dtype=np.int64)[None, :]
    do = np.asarray(dst_off, dtype=np.int64)[:, None] + np.arange(run_elems, dtype=np.int64)[None, :]
    dst.reshape(-1)[do] = src.reshape(-1)[so]


def copy_runs_loops(src: np.ndarray, dst: np.ndarray, src_off, dst_off, run_elems: int):
    """The kernel's formula, element by element (copy_kernel.cu:29-34). Tiny inputs only."""
    s, d = src.reshape(-1), dst.reshape(-1)
    for p in range(len(src_off)):
        src_start, dest_start = int(src_off[p]), int(dst_off[p])
        for elem_idx in range(run_elems):
            d[dest_start + elem_idx] = s[src_start + elem_idx]


# ---------------------------------------------------------------------------------------------
# ring bookkeeping  (copy_kernel.cu:81-89,116-127; ipc_service.cpp:118-138)
# ---------------------------------------------------------------------------------------------
def ring_step_c(ring: Ring, n_pages, page_size, dims, elem_bytes=2) -> int:
    head, kvh, layers, kv = dims
    return clib().oracle_ring_step(C.byref(ring), n_pages, page_size, head, kvh, layers, kv, elem_bytes)


def ring_step_py(state: dict, n_pages, page_size, dims, elem_bytes=2) -> int:
    """state: dict(current_offset, last_valid_offset, buffer_size, ...). Follows the reference line
    by line."""
    head, kvh, layers, kv = dims
    elements_per_token = head * kvh * layers * kv
    page_elements = page_size * elements_per_token
    data_size = n_pages * page_elements * elem_bytes
    if state["current_offset"] + data_size > state["buffer_size"]:
        state["current_offset"] = 0
    at = state["current_offset"]
    state["last_valid_offset"] = state["current_offset"]
    state["current_offset"] += data_size
    state["tensor_dim"] = 5
    state["tensor_shape"] = [n_pages * page_size, head, kvh, layers, kv]
    state["data_size"] = data_size
    return at


def ring_send_c(ring: Ring, data_size: int, shape) -> int:
    sh, shp = _i64(shape)
    return clib().oracle_ring_send(C.byref(ring), data_size, shp, len(sh))


# ---------------------------------------------------------------------------------------------
# offset tables  (kvcache.py:161-174,187-196)
# ---------------------------------------------------------------------------------------------
def build_offsets_loops(cache_pages_list, id_token_pair_list, page_size, scale=1):
    """The reference's two loops, verbatim in structure. scale=1 gives its token-unit numbers."""
    page_indices, page_offsets = [], []
    current_offset = 0
    for idx, page_list in enumerate(cache_pages_list):
        item_token_num = id_token_pair_list[idx][1]
        for page_idx, page in enumerate(page_list):
            size = (item_token_num % page_size) if (page_idx == len(page_list) - 1 and
                                                     item_token_num % page_size != 0) else page_size
            page_indices.append(page)
            page_offsets.append(current_offset)
            current_offset += size
    src_offsets = [p * page_size * scale for p in page_indices]
    dest_offsets = [o * scale for o in page_offsets]
    return src_offsets, dest_offsets, current_offset


def build_offsets_c(cache_pages_list, item_tokens, page_size, scale=1):
    counts = np.array([len(p) for p in cache_pages_list], dtype=np.int64)
    n = int(counts.sum())
    pages = np.concatenate([np.asarray(p, dtype=np.int64) for p in cache_pages_list]) if n else np.zeros(0, np.int64)
    pages, pp = _i64(pages)
    counts, cp = _i64(counts)
    tokens, tp = _i64(item_tokens)
    so = np.zeros(n, dtype=np.int64)
    do = np.zeros(n, dtype=np.int64)
    total = clib().oracle_build_offsets(pp, cp, tp, len(counts), page_size, scale,
                                        so.ctypes.data_as(C.POINTER(C.c_int64)),
                                        do.ctypes.data_as(C.POINTER(C.c_int64)))
    return so, do, total


# ---------------------------------------------------------------------------------------------
# layered gather / scatter
#   pool: numpy array [n_planes, n_pool_pages, tile_elems]; staging: flat array of slots.
# ---------------------------------------------------------------------------------------------
def _plane_ptrs(pool: np.ndarray):
    n_planes = pool.shape[0]
    stride = pool.strides[0]
    arr = (C.c_void_p * n_planes)(*[pool.ctypes.data + q * stride for q in range(n_planes)])
    return arr


def _layered_c(fn, pool, requests, layout, staging):
    assert pool.flags.c_contiguous and pool.ndim == 3
    n_planes, n_pool_pages, tile_elems = pool.shape
    tile_bytes = tile_elems * pool.dtype.itemsize
    ids = np.concatenate([np.asarray(r, dtype=np.int64) for r in requests]) if len(requests) else np.zeros(0, np.int64)
    ids, idp = _i64(ids)
    rp, rpp = _i64([len(r) for r in requests])
    st = _bytes_view(staging)
    assert st.size >= int(rp.sum()) * n_planes * tile_bytes
    return fn(_plane_ptrs(pool), n_planes, n_pool_pages, tile_bytes, tile_bytes, idp, rpp, len(rp),
              0 if layout == "layer_major" else 1, st.ctypes.data)


def gather_layered_c(pool, requests, layout="layer_major"):
    n_planes, _, tile_elems = pool.shape
    total = sum(len(r) for r in requests)
    staging = np.zeros(total * n_planes * tile_elems, dtype=pool.dtype)
    bad = _layered_c(clib().oracle_gather_layered, pool, requests, layout, staging)
    assert bad == 0, f"{bad} page ids out of range"
    return staging


def scatter_layered_c(pool, requests, staging, layout="layer_major"):
    bad = _layered_c(clib().oracle_scatter_layered, pool, requests, layout, staging)
    assert bad == 0, f"{bad} page ids out of range"


def planes_of_token_kv_layers(layers, block_tokens):
    """The Worker's per-layer tensors [blocks*block_tokens, 2, heads, dim] (Worker/Worker.py:74-78)
    restated as the planar pool [2*L, blocks, block_tokens*heads*dim] the layered functions take:
    plane 2*l + k, page b = the block's tokens of K (k = 0) or V (k = 1), token-major. Pure numpy
    reshapes: the statement of the layout, independent of any stride arithmetic."""
    planes = []
    for a in layers:
        slots, two, h, d = a.shape
        assert two == 2 and slots % block_tokens == 0
        blk = a.reshape(slots // block_tokens, block_tokens, 2, h * d)
        for k in (0, 1):
            planes.append(np.ascontiguousarray(blk[:, :, k, :]).reshape(slots // block_tokens, block_tokens * h * d))
    return np.stack(planes)


def token_kv_layers_of_planes(planes, block_tokens, heads, dim):
    """Inverse of planes_of_token_kv_layers: list of [blocks*block_tokens, 2, heads, dim] arrays."""
    n_planes, blocks, _ = planes.shape
    out = []
    for l in range(n_planes // 2):
        a = np.empty((blocks, block_tokens, 2, heads * dim), dtype=planes.dtype)
        for k in (0, 1):
            a[:, :, k, :] = planes[2 * l + k].reshape(blocks, block_tokens, heads * dim)
        out.append(a.reshape(blocks * block_tokens, 2, heads, dim))
    return out


def gather_layered_np(pool, requests, layout="layer_major"):
    """out_r[q][j] = pool[q][ids_r[j]] (layer-major) or out_r[j][q] (page-major), requests packed."""
    parts = []
    for ids in requests:
        ids = np.asarray(ids, dtype=np.int64)
        g = pool[:, ids, :]                       # [planes, m, tile]
        if layout != "layer_major":
            g = np.transpose(g, (1, 0, 2))        # [m, planes, tile]
        parts.append(np.ascontiguousarray(g).reshape(-1))
    return np.concatenate(parts) if parts else np.zeros(0, dtype=pool.dtype)


def scatter_layered_np(pool, requests, staging, layout="layer_major"):
    n_planes, _, tile = pool.shape
    at = 0
    for ids in requests:
        ids = np.asarray(ids, dtype=np.int64)
        m = len(ids)
        blk = staging[at: at + m * n_planes * tile]
        if layout == "layer_major":
            pool[:, ids, :] = blk.reshape(n_planes, m, tile)
        else:
            pool[:, ids, :] = np.transpose(blk.reshape(m, n_planes, tile), (1, 0, 2))
        at += m * n_planes * tile


def gather_layered_loops(pool, requests, layout="layer_major"):
    """Page by page, element by element. Tiny inputs only."""
    n_planes, _, tile = pool.shape
    total = sum(len(r) for r in requests)
    out = np.zeros(total * n_planes * tile, dtype=pool.dtype)
    base = 0
    for ids in requests:
        m = len(ids)
        for q in range(n_planes):
            for j in range(m):
                slot = base + q * m + j if layout == "layer_major" else base + j * n_planes + q
                for e in range(tile):
                    out[slot * tile + e] = pool[q, int(ids[j]), e]
        base += m * n_planes
    return out


# ---------------------------------------------------------------------------------------------
# fused page move + layout change: token-major pages <-> per-layer paged NHD pool
#   tm: numpy array [n_tm_pages, P, D, H, L, 2] (token_shape = (D, H, L, 2), Model/qwen2.py:519-522)
#   layers: list of L numpy arrays, form "token_kv" [blocks*P, 2, H, D] (Worker/Worker.py:74-78) or
#           "block_kv" [blocks, 2, P, H, D] (Model/qwen2.py:532-536)
# ---------------------------------------------------------------------------------------------
def _nhd_strides(layers, form, P):
    if form == "token_kv":
        slots, two, H, D = layers[0].shape
        return slots // P, H, D, (P * 2 * H * D, H * D, 2 * H * D)
    blocks, two, p, H, D = layers[0].shape
    assert p == P
    return blocks, H, D, (2 * P * H * D, P * H * D, H * D)


def transpose_pages_c(layers, form, tm, block_ids, tm_pages, direction):
    """direction "load": tm -> layers; "store": layers -> tm. In place. Returns skipped pages."""
    P = tm.shape[1]
    n_blocks, H, D, (bs, ks, ts) = _nhd_strides(layers, form, P)
    assert tm.shape[2:] == (D, H, len(layers), 2) and tm.flags.c_contiguous
    assert all(a.flags.c_contiguous for a in layers)
    ptrs = (C.c_void_p * len(layers))(*[a.ctypes.data for a in layers])
    b, bp = _i64(block_ids)
    t, tp = _i64(tm_pages)
    return clib().oracle_transpose_pages(ptrs, len(layers), H, D, P, tm.dtype.itemsize, n_blocks, bs, ks, ts,
                                         tm.ctypes.data, tm.shape[0], bp, tp, len(b),
                                         1 if direction == "load" else 0)


def transpose_pages_np(layers, form, tm, block_ids, tm_pages, direction):
    """The same with numpy's transpose: per page and layer, [P, D, H, 2] <-> [P, 2, H, D]."""
    P = tm.shape[1]
    for b, p in zip(block_ids, tm_pages):
        for l, layer in enumerate(layers):
            if form == "token_kv":
                view = layer[b * P:(b + 1) * P]                      # [P, 2, H, D]
                axes_to, axes_from = (0, 3, 2, 1), (0, 3, 2, 1)      # [P,D,H,2] <-> [P,2,H,D]
            else:
                view = layer[b]                                      # [2, P, H, D]
                axes_to, axes_from = (3, 0, 2, 1), (1, 3, 2, 0)      # [P,D,H,2] -> [2,P,H,D] and back
            if direction == "load":
                view[...] = np.transpose(tm[p][:, :, :, l, :], axes_to)
            else:
                tm[p][:, :, :, l, :] = np.transpose(view, axes_from)


# ---------------------------------------------------------------------------------------------
# the reference's CPU path as a torch routine (timed by the benchmark as the CPU baseline)
# ---------------------------------------------------------------------------------------------
def gather_layered_torch(pool_t, ids_t, out_t=None):
    """pool_t: host tensor [n_planes, n_pool_pages, tile]; ids_t: int64 [m]. -> [n_planes, m, tile]."""
    import torch
    return torch.index_select(pool_t, 1, ids_t, out=out_t)


def scatter_layered_torch(pool_t, ids_t, staged_t):
    """pool_t[:, ids] = staged (unique ids)."""
    pool_t.index_copy_(1, ids_t, staged_t)
