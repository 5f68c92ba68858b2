"""Run copy: the reference's generic offset->offset page copy on raw tensors.

copy_runs(src, dst, src_off, dst_off, run_elems) performs, for every i,
    dst.flatten()[dst_off[i] : dst_off[i]+run_elems] = src.flatten()[src_off[i] : src_off[i]+run_elems]
which is block_per_page_copy_kernel (Bi-KV/SharedMemory/CUDA_Shared/copy_kernel.cu:9-36) when src is
a device tensor and zero_copy_page_kernel (copy_kernel.cu:39-66) when src is a pinned host tensor.
Offsets are int64 device tensors in elements, as the reference's callers pass them
(test_page_ipc.py:58-65).
"""
import ctypes as C

import torch

from . import _lib


def _dev_ptr(t: torch.Tensor, what: str):
    if t.is_cuda:
        return t.data_ptr()
    if t.is_pinned():
        return t.data_ptr()  # hipHostMalloc'd memory is mapped at the same address on the device
    raise RuntimeError(f"{what} must be on CUDA or in pinned host memory")


def copy_runs(src: torch.Tensor, dst: torch.Tensor, src_off: torch.Tensor, dst_off: torch.Tensor,
              run_elems: int, device=None, run_lens: torch.Tensor = None, unit_elems: int = 1):
    """`run_lens` (int64 device tensor) makes the runs ragged: run i moves run_lens[i] units, at most
    run_elems elements; `unit_elems` is the unit of offsets and lengths in elements (1 = the
    reference's element offsets; elements per token = the token offsets kvcache.py computes)."""
    if not src.is_contiguous() or not dst.is_contiguous():
        raise RuntimeError("Cache data must be contiguous")
    if src.element_size() != dst.element_size():
        raise RuntimeError("source and destination element sizes differ")
    tables = [("src_offsets", src_off), ("dest_offsets", dst_off)]
    if run_lens is not None:
        tables.append(("run_lens", run_lens))
    for name, t in tables:
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be on CUDA")
        if t.dtype != torch.int64 or not t.is_contiguous() or t.dim() != 1:
            raise RuntimeError(f"{name} must be a contiguous 1-D int64 tensor")
    if src_off.numel() != dst_off.numel():
        raise RuntimeError("src_offsets and dest_offsets differ in length")
    if run_lens is not None and run_lens.numel() != src_off.numel():
        raise RuntimeError("run_lens and src_offsets differ in length")
    dev = torch.device(device) if device is not None else src_off.device
    es = src.element_size()
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    if run_lens is not None:
        with torch.cuda.device(dev):
            _lib.check(_lib.load().bikv_copy_runs_ragged(
                _dev_ptr(src, "source"), src.numel() * es, _dev_ptr(dst, "destination"), dst.numel() * es,
                src_off.data_ptr(), dst_off.data_ptr(), run_lens.data_ptr(), src_off.numel(),
                int(run_elems) * es, int(unit_elems) * es, stream))
        return
    if unit_elems != 1:
        raise RuntimeError("unit_elems other than 1 needs run_lens")
    with torch.cuda.device(dev):
        _lib.check(_lib.load().bikv_copy_runs(
            _dev_ptr(src, "source"), src.numel() * es, _dev_ptr(dst, "destination"), dst.numel() * es,
            src_off.data_ptr(), dst_off.data_ptr(), src_off.numel(), int(run_elems) * es, es,
            C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)))


def check(device):
    """Synchronises the current stream of `device`; raises if a kernel skipped out-of-range runs."""
    dev = torch.device(device)
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    with torch.cuda.device(dev):
        _lib.check(_lib.load().bikv_check_status(idx, C.c_void_p(torch.cuda.current_stream(dev).cuda_stream), None))
