"""Device memory placed for the MI355X memory system (bikv_device_alloc).

The reference allocates its pools with torch (Bi-KV/DistributedStorage/kvcache.py:38-43,
Bi-KV/Worker/Worker.py:74-78). On MI355X where a pool lies physically decides how fast pages can be
scattered into it: the address space behaves as two halves, and random writes confined to one half run
15-18 % slower than the same writes spread over both. DeviceBuffer is memory whose physical chunks
alternate between the halves; `.tensor` is a torch view of it (uint8, or reshaped / re-typed by the
caller) that kernels, torch ops and this library treat like any device tensor.
"""
import contextlib
import ctypes as C

import torch

from . import _lib


class _Span:
    """Exposes device memory to torch without copying; keeps its owner alive as long as torch holds it."""

    def __init__(self, ptr, nbytes, owner):
        self._owner = owner
        self.__cuda_array_interface__ = {"shape": (int(nbytes),), "typestr": "|u1", "data": (int(ptr), False),
                                         "version": 2, "strides": None}


class DeviceBuffer:
    def __init__(self, nbytes: int, device, spread: bool = True, max_filler_bytes: int = None):
        """`max_filler_bytes` bounds the memory the placement may create and release again on its way to
        the second half of HBM (None = the library's default, 96 GiB; < 0 = all free memory but 2 GiB)."""
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("DeviceBuffer needs a GPU (device must be cuda)")
        idx = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        torch.cuda.synchronize(self.device)
        place = _lib.PLACE_SPREAD if spread else _lib.PLACE_SEQUENTIAL
        if max_filler_bytes is None:
            _lib.check(_lib.load().bikv_device_alloc(idx, self.nbytes, place, C.byref(p)))
        else:
            _lib.check(_lib.load().bikv_device_alloc_bounded(idx, self.nbytes, place, int(max_filler_bytes), C.byref(p)))
        self._ptr = p.value
        info = _lib.AllocInfo()
        _lib.check(_lib.load().bikv_device_alloc_info(p, C.byref(info)))
        self.info = {"bytes": info.bytes, "chunk_bytes": info.chunk_bytes, "n_chunks": info.n_chunks,
                     "n_other_half": info.n_other_half, "n_fillers": info.n_fillers, "n_reprobed": info.n_reprobed,
                     "seconds": round(info.seconds, 6), "pair_ms_same": round(info.pair_ms_same, 4),
                     "pair_ms_other": round(info.pair_ms_other, 4)}

    @property
    def tensor(self) -> torch.Tensor:
        """The requested bytes as a uint8 tensor. The tensor keeps this buffer alive."""
        if self._ptr is None:
            raise RuntimeError("DeviceBuffer has been freed")
        return torch.as_tensor(_Span(self._ptr, self.nbytes, self), device=self.device)

    def free(self):
        """Unmaps and releases the memory. Tensors made from it must not be used afterwards."""
        if getattr(self, "_ptr", None) is not None:
            p, self._ptr = self._ptr, None
            _lib.check(_lib.load().bikv_device_free(C.c_void_p(p)))

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def device_empty(nbytes: int, device, spread: bool = True, max_filler_bytes: int = None) -> torch.Tensor:
    """A uint8 device tensor of `nbytes` whose memory came from bikv_device_alloc; it is released when the
    last tensor that views it is gone and the collector has run."""
    return DeviceBuffer(nbytes, device, spread, max_filler_bytes).tensor


_PLACED_POOL = {}


def placed_mem_pool(device=None):
    """A torch.cuda.MemPool (one per device, created on first use) whose segments come from
    bikv_device_alloc instead of hipMalloc. Every segment is a whole number of chunks of at least 256 MiB
    and is placed with a timed probe, so the pool is meant for the few large KV allocations of a process,
    not for its everyday tensors."""
    idx = None if device is None else torch.device(device).index
    if idx is None:
        idx = torch.cuda.current_device()
    if idx not in _PLACED_POOL:
        _lib.load()         # fails loudly when the library has not been built
        alloc = torch.cuda.memory.CUDAPluggableAllocator(_lib.LIB_PATH, "bikv_torch_alloc", "bikv_torch_free")
        pool = torch.cuda.MemPool(alloc.allocator())
        # The pool and its allocator live until the process ends and are never torn down: destroying them while
        # the interpreter finalises releases segments through objects that may already be gone. One extra
        # reference each keeps their destructors from ever running; the driver reclaims the memory at exit.
        for obj in (pool, alloc, alloc.allocator()):
            C.pythonapi.Py_IncRef(C.py_object(obj))
        _PLACED_POOL[idx] = (pool, alloc)
    return _PLACED_POOL[idx][0]


@contextlib.contextmanager
def placed_allocations(device=None):
    """Inside this context torch's allocations on `device` come from bikv_device_alloc, so a caller keeps its
    own allocation code — the reference's `torch.empty((cache_size,) + token_shape, ...)` of
    Bi-KV/DistributedStorage/kvcache.py:38-43 or the per-layer `torch.zeros` of Bi-KV/Worker/Worker.py:74-78 —
    and still gets pools spread over both halves of HBM:

        with bikv_pagecopy.placed_allocations("cuda:0"):
            self.local_kvcache = [torch.zeros(...) for _ in range(num_layers)]

    Allocate only the pools here: every request torch passes on is rounded up to whole 256 MiB chunks.
    The memory returns to the pool when its tensors die and to the device when the process ends."""
    pool = placed_mem_pool(device)
    with torch.cuda.use_mem_pool(pool, device=device):
        yield pool
