"""The Worker-side callers of the KV transfer, as functions.

Mirrors of Worker.receive_kvcache_data_batch (Bi-KV/Worker/Worker.py:162-191) and
Worker.send_kvcache_data_batch (Worker.py:193-218). Both are stubs in the reference: the receiving one
allocates `recv_tensor` and has its `ipc_service.consumer_receive()` / RDMA calls commented out, and nothing
ever moves the received tokens into the model's per-layer paged cache `local_kvcache` (Worker.py:74-78);
the sending one allocates `send_tensor`, leaves its fill from the compute buffer commented out (Worker.py:207)
and sends nothing. These functions do what the stubs outline, with the same inputs:

  `combined_task_info`  the coordinator's message (TaskInfo.proto CombindedTaskInfo): `cache_worker`,
                        `token_num`, `id_token_pair` = [(item id, tokens)]; read as attributes (the protobuf
                        object the Worker gets) or as keys (the dict kvcache.py gets)
  `worker_index`        this Worker's index: a transfer with `cache_worker == worker_index` goes through the
                        shared-memory ring of `ipc_service` (same GPU box), any other through the transport's
                        pinned host region (the reference's RDMA endpoint sends from / lands in host memory,
                        NetworkTransport/onesided_rdma.h:301-337)
  `kv_pool`             the Worker's paged cache as an NHDPool (NHDPool.from_token_kv_layers(local_kvcache, 16))
  `block_ids`           the blocks of that cache the tokens occupy, in token order — what the Worker's page
                        manager hands out (Worker.py:56, DistributedStorage/PageManager.py:105-115):
                        ceil(tokens / block_tokens) ids, unordered, unique

The token-major image [tokens, head_dim, kv_heads, layers, 2] is cut into pages of `block_tokens` tokens and
every page goes through the fused page move + layout change (bikv_nhd_load_token_major /
bikv_nhd_store_token_major): one kernel launch per transfer. Stage timings are kept the way the cache side
keeps them (kvcache_calls.StageTimes; printed when SM_DEBUG is set).
"""
import time
from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np
import torch

import ipc_service

from .kvcache_calls import SM_DEBUG
from .nhd import NHDPool


@dataclass
class WorkerStageTimes:
    """Host wall time of the stages of one Worker-side transfer."""
    tokens: int = 0
    pages: int = 0
    data_bytes: int = 0
    wait_ms: float = 0.0      # receive: blocked in consumer_receive; send: 0
    layout_ms: float = 0.0    # page list upload + layout-change kernel, stream sync included
    publish_ms: float = 0.0   # send through the ring: producer_send (copy into the ring + publication)
    total_ms: float = 0.0

    def report(self, what: str) -> str:
        mb = self.data_bytes / 1024 / 1024
        rate = mb / (self.layout_ms * 1e-3) if self.layout_ms > 0 else 0.0
        return (f"[{what}] {self.tokens} tokens in {self.pages} blocks, {mb:.2f} MB: wait {self.wait_ms:.2f} ms, "
                f"layout change {self.layout_ms:.2f} ms ({rate:.2f} MB/s), publish {self.publish_ms:.2f} ms, "
                f"total {self.total_ms:.2f} ms")


_last_times = WorkerStageTimes()


def last_stage_times() -> WorkerStageTimes:
    """Timings of the most recent receive_ / send_kvcache_data_batch call of this process."""
    return _last_times


def _field(info, name):
    return info[name] if isinstance(info, dict) else getattr(info, name)


def _pair_tokens(pair) -> int:
    if isinstance(pair, (tuple, list)):
        return int(pair[1])
    return int(pair["token_num"] if isinstance(pair, dict) else pair.token_num)


def _token_shape(kv_pool: NHDPool):
    return (kv_pool.head_dim, kv_pool.kv_heads, kv_pool.n_layers, 2)


def _check_blocks(kv_pool: NHDPool, block_ids, tokens: int) -> np.ndarray:
    ids = np.ascontiguousarray(np.asarray(block_ids, dtype=np.int64).reshape(-1))
    need = -(-tokens // kv_pool.block_tokens)
    if ids.size != need:
        raise RuntimeError(f"{tokens} tokens occupy {need} blocks of {kv_pool.block_tokens} tokens, "
                           f"but {ids.size} block ids were given")
    return ids


def _finish(times: WorkerStageTimes, what: str, t_start: float):
    global _last_times
    times.total_ms = (time.perf_counter() - t_start) * 1e3
    _last_times = times
    if SM_DEBUG:
        print(times.report(what), flush=True)


def receive_kvcache_data_batch(combined_task_info, kv_pool: NHDPool, block_ids: Sequence[int], worker_index: int,
                               host_image: Optional[torch.Tensor] = None, timeout_ms: int = -1,
                               release: bool = False) -> int:
    """KV of `token_num` tokens arrives and lands in blocks `block_ids` of the Worker's paged cache.

    Same box (`cache_worker == worker_index`): the tensor comes out of the ring (consumer_receive, the call
    Worker.py:173 has commented out) and goes block by block into the cache; with `release` the ring space is
    handed back afterwards (consumer_release, for producers that run with back-pressure). Other box:
    `host_image` is the pinned host tensor [token_num, head_dim, kv_heads, layers, 2] the transport has
    filled; the kernel reads it over the host link. Returns the number of tokens written. A last block that
    is only partly covered gets zeros in its remaining token slots."""
    t_start = time.perf_counter()
    times = WorkerStageTimes()
    cache_worker = int(_field(combined_task_info, "cache_worker"))
    token_num = int(_field(combined_task_info, "token_num"))
    shape = _token_shape(kv_pool)
    ids = _check_blocks(kv_pool, block_ids, token_num)
    if cache_worker == worker_index:
        recv = ipc_service.consumer_receive(timeout_ms=timeout_ms)
        times.wait_ms = (time.perf_counter() - t_start) * 1e3
        if tuple(recv.shape[1:]) != shape or recv.shape[0] < token_num:
            raise RuntimeError(f"received tensor {tuple(recv.shape)} does not hold {token_num} tokens of shape {shape}")
        image = recv
    else:
        if host_image is None:
            raise RuntimeError("a transfer from another box needs the transport's pinned host image")
        if host_image.is_cuda or not host_image.is_pinned():
            raise RuntimeError("CPU data must be pinned memory")       # message of copy_kernel.cu:142
        if tuple(host_image.shape[1:]) != shape or host_image.shape[0] < token_num:
            raise RuntimeError(f"host image {tuple(host_image.shape)} does not hold {token_num} tokens of shape {shape}")
        image = host_image
    t_layout = time.perf_counter()
    P = kv_pool.block_tokens
    full = token_num // P
    with torch.cuda.device(kv_pool.device):
        if full:
            dev_ids, pages = kv_pool.page_list(ids[:full], check_unique=True)
            kv_pool.load_token_major(image[: full * P].reshape((full, P) + shape), dev_ids, pages)
        tail = token_num - full * P
        if tail:
            # the partly covered last block: its tokens, then zeros, as one page of its own
            page = torch.zeros((1, P) + shape, dtype=kv_pool.dtype, device=kv_pool.device)
            page[0, :tail].copy_(image[full * P: token_num], non_blocking=True)
            dev_ids, pages = kv_pool.page_list(ids[full:])
            kv_pool.load_token_major(page, dev_ids, pages)
        kv_pool.check()                       # stream sync + rejected block ids raise here
    if cache_worker == worker_index and release:
        ipc_service.consumer_release()
    times.layout_ms = (time.perf_counter() - t_layout) * 1e3
    times.tokens, times.pages = token_num, len(ids)
    times.data_bytes = token_num * kv_pool.token_elems * image.element_size()
    _finish(times, "receive_kvcache_data_batch", t_start)
    return token_num


def send_kvcache_data_batch(combined_task_info, kv_pool: NHDPool, block_ids: Sequence[int], worker_index: int,
                            host_image: Optional[torch.Tensor] = None,
                            staging: Optional[torch.Tensor] = None) -> int:
    """The KV of the items in `id_token_pair` leaves the Worker's paged cache in token-major form.

    The number of tokens is the sum over `id_token_pair`, as Worker.py:197-199 computes it; `block_ids` names
    the blocks that hold them, in token order. Same box: the blocks are stored into a device tensor
    (`staging`, [blocks, block_tokens, head_dim, kv_heads, layers, 2], allocated when not given) and
    producer_send publishes its first `tokens` tokens through the ring as [tokens, head_dim, kv_heads, layers,
    2]. Other box: the kernel stores straight into the transport's pinned `host_image` (at least
    blocks*block_tokens tokens long), which the caller then posts. Returns the number of tokens sent."""
    t_start = time.perf_counter()
    times = WorkerStageTimes()
    cache_worker = int(_field(combined_task_info, "cache_worker"))
    total = sum(_pair_tokens(p) for p in _field(combined_task_info, "id_token_pair"))
    shape = _token_shape(kv_pool)
    ids = _check_blocks(kv_pool, block_ids, total)
    P, n = kv_pool.block_tokens, len(ids)
    same_box = cache_worker == worker_index
    if same_box:
        if staging is None:
            staging = torch.empty((n, P) + shape, dtype=kv_pool.dtype, device=kv_pool.device)
        elif not staging.is_cuda or staging.numel() < n * P * kv_pool.token_elems:
            raise RuntimeError("staging must be a device tensor of at least blocks*block_tokens tokens")
        image = staging
    else:
        if host_image is None:
            raise RuntimeError("a transfer to another box needs the transport's pinned host image")
        if host_image.is_cuda or not host_image.is_pinned():
            raise RuntimeError("CPU data must be pinned memory")
        if host_image.numel() < n * P * kv_pool.token_elems:
            raise RuntimeError(f"host image holds {host_image.numel()} elements, {n} blocks need {n * P * kv_pool.token_elems}")
        image = host_image
    pages_view = image.reshape(-1)[: n * P * kv_pool.token_elems].view((n, P) + shape)
    t_layout = time.perf_counter()
    with torch.cuda.device(kv_pool.device):
        if n:
            dev_ids, pages = kv_pool.page_list(ids)
            kv_pool.store_token_major(pages_view, dev_ids, pages)
        kv_pool.check()
    times.layout_ms = (time.perf_counter() - t_layout) * 1e3
    if same_box:
        t_pub = time.perf_counter()
        ipc_service.producer_send(pages_view.view((n * P,) + shape)[:total])
        times.publish_ms = (time.perf_counter() - t_pub) * 1e3
    times.tokens, times.pages = total, n
    times.data_bytes = total * kv_pool.token_elems * image.element_size()
    _finish(times, "send_kvcache_data_batch", t_start)
    return total
