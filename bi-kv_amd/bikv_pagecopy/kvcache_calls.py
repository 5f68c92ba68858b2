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
from typing import Dict, Sequence, Tuple

import torch

import ipc_service

from .offsets import build_run_offsets

# the reference hard-codes these (kvcache.py:198-203, Model/qwen2.py:512-522)
REFERENCE_DIMS = (128, 2, 28, 2)


def _dims(n_pages: int, page_size: int, dims: Sequence[int]):
    d = ipc_service.TensorDims()
    d.total_tokens = n_pages * page_size
    d.head_size, d.num_kv_heads, d.num_layers, d.kv_pair = (int(x) for x in dims)
    return d


def _tables(info: Dict, page_size: int, dims: Sequence[int], pack_partial_pages, device, index_pool=None):
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
    if index_pool is not None and n:
        dev = index_pool.load(off)            # persistent buffers (kvcache.py:60-64), no allocation
    else:
        dev = torch.from_numpy(off).to(device) if n else torch.empty((off.shape[0], 0), dtype=torch.int64, device=device)
    return dev, n, total


def _send(data, info, page_size, dims, pack_partial_pages, device, whole_pages, index_pool=None) -> Tuple[int, int]:
    if pack_partial_pages not in (False, True, "exact"):
        raise ValueError("pack_partial_pages must be False, True or 'exact'")
    off, n, total = _tables(info, page_size, dims, pack_partial_pages, device, index_pool)
    d = _dims(n, page_size, dims)
    if pack_partial_pages == "exact":
        d.total_tokens = total
        ipc_service.producer_copy_tokens(data, off[0], off[1], off[2], page_size, d)
    else:
        whole_pages(data, off[0], off[1], page_size, d)
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
