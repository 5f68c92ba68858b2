"""Layered paged KV pool on one GPU and batched page gather/scatter through libbikv_pagecopy.so.

Host-side mirror of the part of the reference that turns page lists into copy work:
KVCache.shared_data_batch_pages (Bi-KV/DistributedStorage/kvcache.py:132-239) flattens
`cache_pages_list` with two Python loops and uploads two Python lists per call; here the index
arrays of a whole batch of requests are built with numpy and uploaded once, in one tensor.

Pool layouts accepted (plane q = layer*2 + kv):
  * one tensor per plane, each [N, ...] with a contiguous tile per page;
  * one tensor [L, 2, N, ...]                       (planes are slices of one allocation);
  * one tensor per layer [N, 2, ...]                (Bi-KV/Model/qwen2.py:532-536: K and V of a page
                                                     adjacent, page stride = 2 tiles).
"""
import ctypes as C
from typing import List, Optional, Sequence

import numpy as np
import torch

from . import _lib

LAYER_MAJOR = "layer_major"   # request buffer [planes][pages][tile]
PAGE_MAJOR = "page_major"     # request buffer [pages][planes][tile]
_LAYOUT_CODE = {LAYER_MAJOR: _lib.LAYOUT_LAYER_MAJOR, PAGE_MAJOR: _lib.LAYOUT_PAGE_MAJOR}


def _stream_ptr(device):
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class PageBatch:
    """Index arrays of one batch of requests, resident on the device.

    index[0] = page ids, index[1] = first staging slot of each page, index[2] = slot stride between
    consecutive planes of that page. Requests are packed back to back in staging in batch order.
    """

    def __init__(self, index: torch.Tensor, req_pages: np.ndarray, n_planes: int, layout: str):
        self.index = index
        self.req_pages = np.ascontiguousarray(req_pages, dtype=np.int64)
        self.n_planes = int(n_planes)
        self.layout = layout
        self.n_pages = int(self.req_pages.sum())
        self.n_slots = self.n_pages * self.n_planes
        first = np.zeros(len(self.req_pages) + 1, dtype=np.int64)
        np.cumsum(self.req_pages, out=first[1:])
        self.req_first_page = first
        self.req_first_slot = first * self.n_planes

    def desc(self, plane_begin=0, plane_count=0, slot_bias=0) -> _lib.PageBatchDesc:
        d = _lib.PageBatchDesc()
        if self.n_pages:
            d.page_ids = self.index[0].data_ptr()       # rows need not be adjacent (persistent buffers)
            d.slots = self.index[1].data_ptr()
            d.slot_strides = self.index[2].data_ptr()
        d.n_pages = self.n_pages
        d.plane_begin = plane_begin
        d.plane_count = plane_count
        d.slot_bias = slot_bias
        d.layout_hint = _lib.HINT_LAYER_MAJOR if self.layout == LAYER_MAJOR else _lib.HINT_PAGE_MAJOR
        return d

    def request_view(self, staging: torch.Tensor, r: int) -> torch.Tensor:
        """The slots of request r as [planes, pages, tile] (layer-major) or [pages, planes, tile]."""
        m = int(self.req_pages[r])
        s0 = int(self.req_first_slot[r])
        flat = staging.reshape(self.n_slots, -1)[s0:s0 + m * self.n_planes]
        if self.layout == LAYER_MAJOR:
            return flat.reshape(self.n_planes, m, -1)
        return flat.reshape(m, self.n_planes, -1)


def build_index(requests: Sequence[np.ndarray], n_planes: int, layout: str):
    """numpy form of the three index arrays for a list of per-request page-id lists."""
    if layout not in _LAYOUT_CODE:
        raise ValueError(f"unknown layout {layout!r}")
    req_pages = np.fromiter((len(r) for r in requests), dtype=np.int64, count=len(requests))
    n = int(req_pages.sum())
    idx = np.empty((3, n), dtype=np.int64)
    if n:
        idx[0] = np.concatenate([np.asarray(r, dtype=np.int64).reshape(-1) for r in requests])
        first = np.zeros(len(requests), dtype=np.int64)
        np.cumsum(req_pages[:-1], out=first[1:])
        if layout == LAYER_MAJOR:
            within = np.arange(n, dtype=np.int64) - np.repeat(first, req_pages)
            idx[1] = np.repeat(first * n_planes, req_pages) + within
            idx[2] = np.repeat(req_pages, req_pages)
        else:
            idx[1] = np.arange(n, dtype=np.int64) * n_planes
            idx[2] = 1
    return idx, req_pages


class PagedKVPool:
    """A paged KV pool described to the library once; owns the native pool handle."""

    def __init__(self, plane_ptrs: Sequence[int], n_pages: int, tile_bytes: int,
                 page_stride_bytes: int, device, dtype=torch.uint8,
                 scale_plane_ptrs: Optional[Sequence[int]] = None, scale_tile_bytes: int = 0,
                 scale_page_stride_bytes: int = 0, keepalive=None, row_bytes: int = 0,
                 row_stride_bytes: int = 0):
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("PagedKVPool needs a GPU pool (device must be cuda)")
        self.n_planes = len(plane_ptrs)
        self.n_pages = int(n_pages)
        self.tile_bytes = int(tile_bytes)
        self.page_stride_bytes = int(page_stride_bytes)
        self.scale_tile_bytes = int(scale_tile_bytes)
        self.dtype = dtype
        self._keepalive = keepalive
        lib = _lib.load()
        d = _lib.PoolDesc()
        d.device = self.device.index if self.device.index is not None else torch.cuda.current_device()
        d.n_planes = self.n_planes
        d.n_pages = self.n_pages
        d.tile_bytes = self.tile_bytes
        d.page_stride_bytes = self.page_stride_bytes
        d.row_bytes = int(row_bytes)
        d.row_stride_bytes = int(row_stride_bytes)
        arr = (C.c_void_p * self.n_planes)(*[int(p) for p in plane_ptrs])
        d.plane_base = C.cast(arr, C.POINTER(C.c_void_p))
        if scale_plane_ptrs is not None:
            if len(scale_plane_ptrs) != self.n_planes:
                raise RuntimeError("scale planes must match payload planes one to one")
            sarr = (C.c_void_p * self.n_planes)(*[int(p) for p in scale_plane_ptrs])
            d.scale_plane_base = C.cast(sarr, C.POINTER(C.c_void_p))
            d.scale_tile_bytes = int(scale_tile_bytes)
            d.scale_page_stride_bytes = int(scale_page_stride_bytes)
        self._device_index = d.device
        h = C.c_void_p()
        _lib.check(lib.bikv_pool_create(C.byref(d), C.byref(h)))
        self._h = h

    # ---- constructors from tensors ----------------------------------------------------------
    @staticmethod
    def _check_plane(t: torch.Tensor):
        if not t.is_cuda:
            raise RuntimeError("Cache data must be on CUDA")  # message of copy_kernel.cu:78
        if not t.is_contiguous():
            raise RuntimeError("Cache data must be contiguous")  # copy_kernel.cu:79

    @classmethod
    def from_planes(cls, planes: Sequence[torch.Tensor], scale_planes: Optional[Sequence[torch.Tensor]] = None):
        """planes[q] is [N, ...]: one contiguous tile per page."""
        for t in planes:
            cls._check_plane(t)
        p0 = planes[0]
        n = p0.shape[0]
        tile = p0[0].numel() * p0.element_size()
        if any(t.shape != p0.shape or t.dtype != p0.dtype for t in planes):
            raise RuntimeError("all planes must share shape and dtype")
        kw = {}
        if scale_planes is not None:
            for t in scale_planes:
                cls._check_plane(t)
            s0 = scale_planes[0]
            if any(t.shape != s0.shape or t.dtype != s0.dtype for t in scale_planes) or s0.shape[0] != n:
                raise RuntimeError("scale planes must share shape and dtype and have one row per page")
            st = s0[0].numel() * s0.element_size()
            kw = dict(scale_plane_ptrs=[t.data_ptr() for t in scale_planes], scale_tile_bytes=st,
                      scale_page_stride_bytes=st)
        return cls([t.data_ptr() for t in planes], n, tile, tile, p0.device, p0.dtype,
                   keepalive=(list(planes), list(scale_planes) if scale_planes is not None else None), **kw)

    @classmethod
    def from_stacked(cls, pool: torch.Tensor, plane_dims: int = 2, scale: Optional[torch.Tensor] = None):
        """pool is [L, 2, N, ...] (plane_dims=2) or [planes, N, ...] (plane_dims=1); scale likewise."""
        cls._check_plane(pool)
        planes = pool.reshape((-1,) + tuple(pool.shape[plane_dims:]))
        splanes = None
        if scale is not None:
            cls._check_plane(scale)
            sp = scale.reshape((-1,) + tuple(scale.shape[plane_dims:]))
            splanes = [sp[q] for q in range(sp.shape[0])]
        return cls.from_planes([planes[q] for q in range(planes.shape[0])], splanes)

    @classmethod
    def from_token_kv_layers(cls, layers: Sequence[torch.Tensor], block_tokens: int):
        """layers[l] is [blocks*block_tokens, 2, heads, dim] as the Worker holds its cache
        (Bi-KV/Worker/Worker.py:74-78): K and V interleave token by token, so the tile of (page, K|V) is
        block_tokens rows of heads*dim elements, two rows apart. Plane q = 2*l + k."""
        for t in layers:
            cls._check_plane(t)
        t0 = layers[0]
        if t0.dim() != 4 or t0.shape[1] != 2 or t0.shape[0] % block_tokens:
            raise RuntimeError("expected [blocks*block_tokens, 2, heads, dim] per layer")
        if any(t.shape != t0.shape or t.dtype != t0.dtype for t in layers):
            raise RuntimeError("all layers must share shape and dtype")
        es = t0.element_size()
        row = t0.shape[2] * t0.shape[3] * es
        ptrs = [t.data_ptr() + k * row for t in layers for k in (0, 1)]
        return cls(ptrs, t0.shape[0] // block_tokens, block_tokens * row, block_tokens * 2 * row, t0.device,
                   dtype=t0.dtype, keepalive=list(layers), row_bytes=row, row_stride_bytes=2 * row)

    @classmethod
    def from_layers_kv_adjacent(cls, layers: Sequence[torch.Tensor]):
        """layers[l] is [N, 2, ...] as in Bi-KV/Model/qwen2.py:532-536."""
        for t in layers:
            cls._check_plane(t)
        t0 = layers[0]
        if t0.shape[1] != 2:
            raise RuntimeError("expected [pages, 2, ...] per layer")
        tile = t0[0, 0].numel() * t0.element_size()
        ptrs = []
        for t in layers:
            if t.shape != t0.shape or t.dtype != t0.dtype:
                raise RuntimeError("all layers must share shape and dtype")
            ptrs += [t.data_ptr(), t.data_ptr() + tile]
        return cls(ptrs, t0.shape[0], tile, 2 * tile, t0.device, t0.dtype, keepalive=list(layers))

    # ---- batches ----------------------------------------------------------------------------
    def make_batch(self, requests: Sequence[Sequence[int]], layout: str = LAYER_MAJOR, index_pool=None,
                   check_unique: bool = False) -> PageBatch:
        """Builds and uploads the index arrays of a batch. With `index_pool` (offsets.RunIndexPool, 3 rows)
        they go into its persistent device buffers through its pinned mirror: no allocation, no upload
        from pageable memory; the batch is then valid until the pool's next load().
        `check_unique=True` (for a batch that will be SCATTERED) raises RuntimeError naming the first page
        id that appears twice: duplicate destinations are a data race on the device."""
        idx, req_pages = build_index(requests, self.n_planes, layout)
        if check_unique:
            _lib.require_unique(idx[0], "scatter batch")
        if index_pool is not None and idx.size:
            dev = index_pool.load(idx)
        else:
            dev = torch.from_numpy(idx).to(self.device) if idx.size else torch.empty((3, 0), dtype=torch.int64, device=self.device)
        return PageBatch(dev, req_pages, self.n_planes, layout)

    def empty_staging(self, batch: PageBatch):
        st = torch.empty(batch.n_slots * self.tile_bytes, dtype=torch.uint8, device=self.device)
        sc = None
        if self.scale_tile_bytes:
            sc = torch.empty(batch.n_slots * self.scale_tile_bytes, dtype=torch.uint8, device=self.device)
        return st, sc

    def _move(self, fn, batch, staging, scale_staging):
        if batch.n_planes != self.n_planes:
            raise RuntimeError("batch was built for a pool with a different number of planes")
        for t in (staging, scale_staging):
            if t is not None and not t.is_contiguous():
                raise RuntimeError("staging buffers must be contiguous")
        if staging.device != self.device:
            raise RuntimeError("staging buffer must be on the pool's device")
        if self.scale_tile_bytes and scale_staging is None:
            raise RuntimeError("pool has scales: a scale staging buffer is required")
        d = batch.desc()
        sp = scale_staging.data_ptr() if scale_staging is not None else None
        sb = scale_staging.numel() * scale_staging.element_size() if scale_staging is not None else 0
        with torch.cuda.device(self.device):
            _lib.check(fn(self._h, C.byref(d), staging.data_ptr(),
                          staging.numel() * staging.element_size(), sp, sb, _stream_ptr(self.device)))

    def gather(self, batch: PageBatch, staging: Optional[torch.Tensor] = None,
               scale_staging: Optional[torch.Tensor] = None):
        """pool -> staging on the current stream (asynchronous). Returns (staging, scale_staging)."""
        if staging is None:
            staging, sc = self.empty_staging(batch)
            if scale_staging is None:
                scale_staging = sc
        self._move(_lib.load().bikv_gather_pages, batch, staging, scale_staging)
        return staging, scale_staging

    def scatter(self, batch: PageBatch, staging: torch.Tensor, scale_staging: Optional[torch.Tensor] = None):
        """staging -> pool on the current stream (asynchronous). Page ids must be unique."""
        self._move(_lib.load().bikv_scatter_pages, batch, staging, scale_staging)

    def check(self):
        """Synchronises the current stream and raises if a kernel rejected a page id or slot."""
        with torch.cuda.device(self.device):
            _lib.check(_lib.load().bikv_check_status(self._device_index, _stream_ptr(self.device), None))

    def close(self):
        if getattr(self, "_h", None):
            _lib.load().bikv_pool_destroy(self._h)
            self._h = None
        self._keepalive = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
