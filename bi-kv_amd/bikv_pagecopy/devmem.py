"""Device memory placed for the MI355X memory system (bikv_device_alloc).

The reference allocates its pools with torch (Bi-KV/DistributedStorage/kvcache.py:38-43,
Bi-KV/Worker/Worker.py:74-78). On MI355X where a pool lies physically decides how fast pages can be
scattered into it: the address space behaves as two halves, and random writes confined to one half run
15-18 % slower than the same writes spread over both. DeviceBuffer is memory whose physical chunks
alternate between the halves; `.tensor` is a torch view of it (uint8, or reshaped / re-typed by the
caller) that kernels, torch ops and this library treat like any device tensor.
"""
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
