"""bikv_pagecopy — host side of the MI355X KV page-copy path (gather / scatter / host staging).

Thin Python over libbikv_pagecopy.so (HIP, gfx950). PyTorch supplies device memory and streams only.
"""
from . import _lib
from ._lib import load, require_unique, reset_tuning, set_tuning
from .devmem import DeviceBuffer, device_empty, placed_allocations, placed_mem_pool
from .nhd import NHDPool
from .offsets import RunIndexPool, build_run_offsets
from .pool import LAYER_MAJOR, PAGE_MAJOR, PageBatch, PagedKVPool, build_index
from .runs import copy_runs
from .staging import HostStager, gather_to_host_noalloc, measure_d2h, measure_h2d, pinned_empty, plan_chunks

__all__ = [
    "load", "DeviceBuffer", "device_empty", "placed_allocations", "placed_mem_pool", "set_tuning", "reset_tuning", "require_unique", "build_run_offsets", "RunIndexPool", "LAYER_MAJOR", "PAGE_MAJOR", "PageBatch", "PagedKVPool",
    "build_index", "copy_runs", "NHDPool", "HostStager", "gather_to_host_noalloc", "measure_d2h", "measure_h2d", "pinned_empty", "plan_chunks",
]
