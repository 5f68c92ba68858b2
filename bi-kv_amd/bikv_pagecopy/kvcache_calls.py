"""The cache-side callers of the page copy, as functions.

Mirrors of KVCache.shared_data_batch_pages (Bi-KV/DistributedStorage/kvcache.py:132-239) and
KVCache.shared_data_batch_pages_cpu2gpu (kvcache.py:241-366): take the coordinator's
`combined_task_info` (`id_token_pair` = [(item id, tokens)], `cache_pages_list` = [[page ids]]),
turn the page lists into offset tables, and hand them to `ipc_service.producer_copy_pages` /
`producer_zero_copy_pages`, which copy into the consumer's ring and publish the shape
`[pages*page_size, head, kv_heads, layers, 2]`.

Differences from the reference's methods, each for a stated reason:
  * offsets are in ELEMENTS (the kernel's unit, copy_kernel.cu:22-33; the reference computes tokens,
    kvcache.py:187-196, which the kernel would misread);
  * the tables are built vectorised and uploaded once (the reference: two Python loops and two
    `torch.tensor(list)` uploads per call);
  * destination offsets are whole pages apart by default, matching the published shape. The
    reference packs a partial last page tighter (kvcache.py:169-174) while still copying whole
    pages, so consecutive destinations overlap and the result depends on execution order;
    `pack_partial_pages=True` reproduces those offsets literally, and
    `pack_partial_pages="exact"` packs the same way but copies only the tail tokens of a partial
    page (ipc_service.producer_copy_tokens), so the consumer receives exactly sum(tokens) tokens.
"""
import os
import time
from dataclasses import dataclass
from typing import Dict, Sequence, Tuple

import torch

import ipc_service

from .offsets import build_run_offsets

# The reference prints per-stage timings of every transfer under a module constant SM_DEBUG
# (kvcache.py:22, printed at :140-238: index building, tensor upload, IPC copy with MB/s, total). Here
# the same figures are always collected (see StageTimes / last_stage_times) and printed when the
# environment variable SM_DEBUG is set to something other than 0.
SM_DEBUG = os.environ.get("SM_DEBUG", "0") not in ("", "0")


@dataclass
class StageTimes:
    """Host wall time of the stages of one transfer, in the reference's own split (kvcache.py:142-238)."""
    pages: int = 0
    tokens: int = 0
    data_bytes: int = 0
    index_ms: float = 0.0     # page lists -> offset tables        (reference: stage 2, :159-179)
    upload_ms: float = 0.0    # tables -> device tensors            (reference: stage 3, :181-207)
    copy_ms: float = 0.0      # producer copy incl. stream sync     (reference: stage 4, :217-231)
    total_ms: float = 0.0

    @property
    def copy_MBps(self) -> float:
        """MiB/s of the copy stage, the unit the reference prints (kvcache.py:230-231)."""
        return self.data_bytes / (self.copy_ms * 1e-3) / 1024 / 1024 if self.copy_ms > 0 else 0.0

    def report(self) -> str:
        per_tok = self.total_ms / self.tokens if self.tokens else 0.0
        return (f"[stage 2] offset tables: {self.index_ms:.2f} ms ({self.pages} pages, {self.tokens} tokens)\n"
                f"[stage 3] upload: {self.upload_ms:.2f} ms\n"
                f"[stage 4] IPC page copy: {self.copy_ms:.2f} ms, {self.data_bytes / 1024 / 1024:.2f} MB, "
                f"{self.copy_MBps:.2f} MB/s\n"
                f"[stage 5] total: {self.total_ms:.2f} ms, {per_tok:.4f} ms per token")


_last_times = StageTimes()


def last_stage_times() -> StageTimes:
    """Timings of the most recent shared_data_batch_pages[_cpu2gpu] call of this process."""
    return _last_times

# the reference hard-codes these (kvcache.py:198-203, Model/qwen2.py:512-522)
REFERENCE_DIMS = (128, 2, 28, 2)


def _dims(n_pages: int, page_size: int, dims: Sequence[int]):
    d = ipc_service.TensorDims()
    d.total_tokens = n_pages * page_size
    d.head_size, d.num_kv_heads, d.num_layers, d.kv_pair = (int(x) for x in dims)
    return d


def _tables(info: Dict, page_size: int, dims: Sequence[int], pack_partial_pages, device, index_pool=None,
            times: StageTimes = None):
    t0 = time.perf_counter()
    pages_list = info["cache_pages_list"]
    tokens = [int(p[1]) for p in info["id_token_pair"]]
    ept = int(dims[0]) * int(dims[1]) * int(dims[2]) * int(dims[3])
    if pack_partial_pages == "exact":
        off, total = build_run_offsets(pages_list, tokens, page_size, unit="tokens", with_sizes=True)
    else:
        off, _ = build_run_offsets(pages_list, tokens, page_size, elements_per_token=ept)
        total = off.shape[1] * page_size
    n = off.shape[1]
    if not pack_partial_pages and n:
        off[1] = range(0, n * page_size * ept, page_size * ept)
    t1 = time.perf_counter()
    if index_pool is not None and n:
        dev = index_pool.load(off)            # persistent buffers (kvcache.py:60-64), no allocation
    else:
        dev = torch.from_numpy(off).to(device) if n else torch.empty((off.shape[0], 0), dtype=torch.int64, device=device)
    if times is not None:
        times.index_ms = (t1 - t0) * 1e3
        times.upload_ms = (time.perf_counter() - t1) * 1e3
    return dev, n, total


def _send(data, info, page_size, dims, pack_partial_pages, device, whole_pages, index_pool=None) -> Tuple[int, int]:
    if pack_partial_pages not in (False, True, "exact"):
        raise ValueError("pack_partial_pages must be False, True or 'exact'")
    global _last_times
    times = StageTimes()
    t_start = time.perf_counter()
    off, n, total = _tables(info, page_size, dims, pack_partial_pages, device, index_pool, times)
    d = _dims(n, page_size, dims)
    t_copy = time.perf_counter()
    if pack_partial_pages == "exact":
        d.total_tokens = total
        ipc_service.producer_copy_tokens(data, off[0], off[1], off[2], page_size, d)
    else:
        whole_pages(data, off[0], off[1], page_size, d)
    t_end = time.perf_counter()     # the producer calls return after their stream synchronise
    times.pages, times.tokens = n, total
    ept = int(dims[0]) * int(dims[1]) * int(dims[2]) * int(dims[3])
    times.data_bytes = total * ept * data.element_size()
    times.copy_ms = (t_end - t_copy) * 1e3
    times.total_ms = (t_end - t_start) * 1e3
    _last_times = times
    if SM_DEBUG:
        print(times.report(), flush=True)
    return n, total


def shared_data_batch_pages(cuda_cache_data: torch.Tensor, combined_task_info: Dict, page_size: int,
                            dims: Sequence[int] = REFERENCE_DIMS,
                            pack_partial_pages=False, index_pool=None) -> Tuple[int, int]:
    """Device pool -> consumer ring. Returns (pages copied, tokens published). `index_pool` (a
    RunIndexPool) keeps the offset tables in persistent device buffers."""
    if not cuda_cache_data.is_cuda:
        raise RuntimeError("Cache data must be on CUDA")
    return _send(cuda_cache_data, combined_task_info, page_size, dims, pack_partial_pages,
                 cuda_cache_data.device, ipc_service.producer_copy_pages, index_pool)


def shared_data_batch_pages_cpu2gpu(cpu_cache_data: torch.Tensor, combined_task_info: Dict, page_size: int,
                                    device, dims: Sequence[int] = REFERENCE_DIMS,
                                    pack_partial_pages=False, index_pool=None) -> Tuple[int, int]:
    """Pinned host pool -> consumer ring, the GPU reading host memory directly (kvcache.py:241-366)."""
    if cpu_cache_data.is_cuda or not cpu_cache_data.is_pinned():
        raise RuntimeError("CPU data must be pinned memory")
    return _send(cpu_cache_data, combined_task_info, page_size, dims, pack_partial_pages,
                 torch.device(device), ipc_service.producer_zero_copy_pages, index_pool)
