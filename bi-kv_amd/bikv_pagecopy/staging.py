"""Device -> pinned-host staging of gathered pages.

The reference stages outgoing KV in host tensors allocated per call (Bi-KV/DistributedStorage/
kvcache.py:105-108, Bi-KV/Worker/Worker.py:203-206) which the RDMA endpoint then sends from a
pinned region (Bi-KV/NetworkTransport/onesided_rdma.h:301-337). HostStager fills such a pinned
region straight from the paged pool: pieces are gathered into per-stream HBM buffers and copied out
with hipMemcpyAsync, several streams in flight (mode "pipelined"), or the gather kernel stores
directly into the mapped pinned buffer (mode "direct"). Each transfer also exists in an enqueue-only
form, so that requests follow each other on the link without a drain in between.
"""
import ctypes as C

import numpy as np
import torch

from . import _lib
from .pool import PagedKVPool, PageBatch, _LAYOUT_CODE

_MODES = {"pipelined": _lib.STAGE_PIPELINED, "direct": _lib.STAGE_DIRECT, "auto": _lib.STAGE_AUTO,
          "pipelined_kernel": _lib.STAGE_PIPELINED_KERNEL}


def pinned_empty(nbytes: int) -> torch.Tensor:
    """A pinned host byte buffer (torch allocates it with hipHostMalloc)."""
    return torch.empty(int(nbytes), dtype=torch.uint8, pin_memory=True)


class HostStager:
    """`n_buffers` lanes (HIP stream + HBM buffer of `chunks_per_launch` x `chunk_bytes`). Mode "auto"
    sends with the kernel storing straight into the pinned image ("direct", a steady ~55.7 GB/s) and
    receives through the DMA engine ("pipelined"): a hipMemcpyAsync device -> host behind a kernel is run by
    the HIP runtime as a shader copy of its own, whose rate has been seen to start at 35 GB/s for seconds.
    The defaults (two copies of 16 MiB per kernel launch, two lanes) measured 98.8 % of a plain pinned
    copy host -> device; 8 MiB x 4 gives 97.7 %, 4 MiB x 4 95.6 %."""

    def __init__(self, device, chunk_bytes: int = 16 << 20, n_buffers: int = 2, chunks_per_launch: int = 2):
        self.device = torch.device(device)
        self.chunk_bytes = int(chunk_bytes)
        self.n_buffers = int(n_buffers)
        self.chunks_per_launch = int(chunks_per_launch)
        idx = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self._device_index = idx
        self._keep = []          # what in-flight asynchronous calls still read
        h = C.c_void_p()
        _lib.check(_lib.load().bikv_stager_create(idx, self.chunk_bytes, self.chunks_per_launch, self.n_buffers,
                                                  C.byref(h)))
        self._h = h

    def _args(self, pool: PagedKVPool, batch: PageBatch, host, mode, host_scale):
        if mode not in _MODES:
            raise ValueError(f"unknown mode {mode!r}")
        for t in (host, host_scale):
            if t is None:
                continue
            if t.is_cuda or not t.is_pinned():
                raise RuntimeError("CPU data must be pinned memory")  # message of copy_kernel.cu:142
            if not t.is_contiguous():
                raise RuntimeError("host staging buffer must be contiguous")
        if pool.scale_tile_bytes and host_scale is None:
            raise RuntimeError("pool has scales: a pinned host_scale buffer is required")
        d = batch.desc()
        rp = batch.req_pages.ctypes.data_as(C.POINTER(C.c_int64))
        return (self._h, pool._h, C.byref(d), rp, len(batch.req_pages), _LAYOUT_CODE[batch.layout],
                host.data_ptr(), host.numel() * host.element_size(),
                host_scale.data_ptr() if host_scale is not None else None,
                host_scale.numel() * host_scale.element_size() if host_scale is not None else 0,
                _MODES[mode]), d

    def _stage(self, entry: str, pool, batch, host, mode, host_scale):
        args, d = self._args(pool, batch, host, mode, host_scale)
        # work queued on the caller's stream (e.g. the upload of the index arrays) must be visible
        torch.cuda.current_stream(self.device).synchronize()
        stats = _lib.StageStats()
        _lib.check(getattr(_lib.load(), entry)(*args, C.byref(stats)))
        self._keep.clear()
        return stats.bytes, stats.n_chunks, stats.wall_seconds

    def _stage_async(self, entry: str, pool, batch, host, mode, host_scale):
        args, d = self._args(pool, batch, host, mode, host_scale)
        stream = C.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)
        _lib.check(getattr(_lib.load(), entry)(*args, stream))
        self._keep.append((pool, batch, host, host_scale))

    def gather_to_host(self, pool: PagedKVPool, batch: PageBatch, host: torch.Tensor, mode: str = "auto",
                       host_scale: torch.Tensor = None):
        """Fills `host` (pinned) with the staging image of `batch` (and `host_scale` with the scale
        image of an fp8 pool); returns (bytes, host copies, seconds)."""
        return self._stage("bikv_gather_to_host", pool, batch, host, mode, host_scale)

    def scatter_from_host(self, pool: PagedKVPool, batch: PageBatch, host: torch.Tensor, mode: str = "auto",
                          host_scale: torch.Tensor = None):
        """Writes the staging image held in `host` (pinned; `host_scale` for an fp8 pool) into the
        pool pages `batch` names (unique ids); returns (bytes, host copies, seconds)."""
        return self._stage("bikv_scatter_from_host", pool, batch, host, mode, host_scale)

    def gather_to_host_async(self, pool: PagedKVPool, batch: PageBatch, host: torch.Tensor, mode: str = "auto",
                             host_scale: torch.Tensor = None):
        """Enqueues the transfer behind the current stream's work and returns; wait() completes it.
        Host images of calls in flight together must not overlap."""
        self._stage_async("bikv_gather_to_host_async", pool, batch, host, mode, host_scale)

    def scatter_from_host_async(self, pool: PagedKVPool, batch: PageBatch, host: torch.Tensor, mode: str = "auto",
                                host_scale: torch.Tensor = None):
        self._stage_async("bikv_scatter_from_host_async", pool, batch, host, mode, host_scale)

    def wait(self):
        """Drains the lanes; returns (bytes, host copies, seconds) of everything enqueued since the
        previous wait and raises if a kernel skipped out-of-range work."""
        stats = _lib.StageStats()
        try:
            _lib.check(_lib.load().bikv_stager_wait(self._h, C.byref(stats)))
        finally:
            self._keep.clear()
        return stats.bytes, stats.n_chunks, stats.wall_seconds

    def trace(self, max_steps: int):
        """Switches the per-step trace on (up to `max_steps` kernel launches and host copies, each between two
        timing events on its lane) or, with 0, off. A diagnostic: it costs a few percent of throughput."""
        _lib.check(_lib.load().bikv_stager_trace(self._h, int(max_steps)))

    def trace_read(self):
        """The steps recorded since trace(n), in issue order, as a list of dicts {lane, kind, bytes, start_ms,
        end_ms}; times count from the start of the first recorded step. Call after wait()."""
        lib = _lib.load()
        n = _lib.check(lib.bikv_stager_trace_read(self._h, None, 0))
        if n == 0:
            return []
        buf = (_lib.TraceStep * n)()
        _lib.check(lib.bikv_stager_trace_read(self._h, buf, n))
        return [{"lane": s.lane, "kind": _lib.TRACE_KINDS[s.kind], "bytes": s.bytes, "start_ms": s.start_ms,
                 "end_ms": s.end_ms} for s in buf]

    def close(self):
        if getattr(self, "_h", None):
            _lib.load().bikv_stager_destroy(self._h)
            self._h = None
        self._keep = []

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def gather_to_host_noalloc(pool: PagedKVPool, batch: PageBatch, host: torch.Tensor, host_scale: torch.Tensor = None):
    """bikv_gather_to_host_noalloc: the pipelined pool -> pinned host transfer for callers that cannot
    allocate. One lane, the current stream, staged through a static scratch array inside the library
    (tiles of at most 16 MiB, scale tiles of at most 64 KiB). Enqueue only: synchronise the stream (or
    call pool.check()) before reading `host`. Calls that overlap in time on one GPU race on the scratch."""
    for t in (host, host_scale):
        if t is None:
            continue
        if t.is_cuda or not t.is_pinned():
            raise RuntimeError("CPU data must be pinned memory")
        if not t.is_contiguous():
            raise RuntimeError("host staging buffer must be contiguous")
    if pool.scale_tile_bytes and host_scale is None:
        raise RuntimeError("pool has scales: a pinned host_scale buffer is required")
    d = batch.desc()
    rp = batch.req_pages.ctypes.data_as(C.POINTER(C.c_int64))
    with torch.cuda.device(pool.device):
        _lib.check(_lib.load().bikv_gather_to_host_noalloc(
            pool._h, C.byref(d), rp, len(batch.req_pages), _LAYOUT_CODE[batch.layout],
            host.data_ptr(), host.numel() * host.element_size(),
            host_scale.data_ptr() if host_scale is not None else None,
            host_scale.numel() * host_scale.element_size() if host_scale is not None else 0,
            C.c_void_p(torch.cuda.current_stream(pool.device).cuda_stream)))


def plan_chunks(req_pages, n_planes: int, layout: str, max_slots: int) -> np.ndarray:
    """The chunk plan of the pipelined mode as an [n_chunks, 6] int64 array:
    (first_page, n_pages, plane_begin, plane_count, first_slot, n_slots). Pure host logic."""
    lib = _lib.load()
    rp = np.ascontiguousarray(req_pages, dtype=np.int64)
    ptr = rp.ctypes.data_as(C.POINTER(C.c_int64))
    n = _lib.check(lib.bikv_plan_chunks(ptr, len(rp), n_planes, _LAYOUT_CODE[layout], max_slots, None, 0))
    out = np.zeros((max(n, 1), 6), dtype=np.int64)
    _lib.check(lib.bikv_plan_chunks(ptr, len(rp), n_planes, _LAYOUT_CODE[layout], max_slots,
                                    out.ctypes.data_as(C.POINTER(C.c_int64)), n))
    return out[:n]


def measure_d2h(device, host: torch.Tensor, dev: torch.Tensor, chunk_bytes: int = 0) -> float:
    """Seconds for a plain hipMemcpyAsync of dev -> host (pinned): the host-link yardstick."""
    idx = torch.device(device).index or 0
    nbytes = min(host.numel() * host.element_size(), dev.numel() * dev.element_size())
    sec = C.c_double()
    torch.cuda.synchronize(device)
    _lib.check(_lib.load().bikv_d2h_copy(idx, host.data_ptr(), dev.data_ptr(), nbytes, chunk_bytes, C.byref(sec)))
    return sec.value


def measure_h2d(device, dev: torch.Tensor, host: torch.Tensor, chunk_bytes: int = 0) -> float:
    """Seconds for a plain hipMemcpyAsync of host (pinned) -> dev."""
    idx = torch.device(device).index or 0
    nbytes = min(host.numel() * host.element_size(), dev.numel() * dev.element_size())
    sec = C.c_double()
    torch.cuda.synchronize(device)
    _lib.check(_lib.load().bikv_h2d_copy(idx, dev.data_ptr(), host.data_ptr(), nbytes, chunk_bytes, C.byref(sec)))
    return sec.value
