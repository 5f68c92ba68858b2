"""Per-layer paged NHD pool (the layout the model reads) and the fused layout change to and from
token-major pages (the layout Bi-KV stores and transfers).

The reference has both layouts and no code between them: Worker.receive_kvcache_data_batch stops at
the received `(token_num,) + token_shape` tensor (Bi-KV/Worker/Worker.py:162-191) and nothing writes
it into `local_kvcache` (Worker.py:74-78); send_kvcache_data_batch allocates the outgoing tensor and
never fills it from the pool (Worker.py:193-207). `load_token_major` / `store_token_major` are those
two missing steps, each one kernel launch over a batch of pages.
"""
import ctypes as C
from typing import Optional, Sequence

import torch

from . import _lib


class NHDPool:
    """L layer tensors addressed (block, kv, token, head, d) with head_dim contiguous."""

    def __init__(self, layers: Sequence[torch.Tensor], block_tokens: int, kv_heads: int, head_dim: int,
                 n_blocks: int, block_stride: int, kv_stride: int, token_stride: int):
        t0 = layers[0]
        for t in layers:
            if not t.is_cuda:
                raise RuntimeError("Cache data must be on CUDA")
            if not t.is_contiguous():
                raise RuntimeError("Cache data must be contiguous")
            if t.shape != t0.shape or t.dtype != t0.dtype:
                raise RuntimeError("all layers must share shape and dtype")
        self.device = t0.device
        self.dtype = t0.dtype
        self.n_layers = len(layers)
        self.kv_heads, self.head_dim, self.block_tokens, self.n_blocks = kv_heads, head_dim, block_tokens, n_blocks
        self.token_elems = head_dim * kv_heads * self.n_layers * 2        # one token, token-major
        self.page_elems = block_tokens * self.token_elems
        self._layers = list(layers)
        d = _lib.NHDDesc()
        d.device = self.device.index if self.device.index is not None else torch.cuda.current_device()
        d.n_layers, d.kv_heads, d.head_dim, d.block_tokens = self.n_layers, kv_heads, head_dim, block_tokens
        d.elem_bytes = t0.element_size()
        d.n_blocks = n_blocks
        d.block_stride_elems, d.kv_stride_elems, d.token_stride_elems = block_stride, kv_stride, token_stride
        arr = (C.c_void_p * self.n_layers)(*[t.data_ptr() for t in layers])
        d.layer_base = C.cast(arr, C.POINTER(C.c_void_p))
        h = C.c_void_p()
        _lib.check(_lib.load().bikv_nhd_create(C.byref(d), C.byref(h)))
        self._h = h

    @classmethod
    def from_token_kv_layers(cls, layers: Sequence[torch.Tensor], block_tokens: int):
        """layers[l] is [blocks*block_tokens, 2, heads, dim] (Bi-KV/Worker/Worker.py:74-78)."""
        slots, two, h, d = layers[0].shape
        if two != 2 or slots % block_tokens:
            raise RuntimeError("expected [blocks*block_tokens, 2, heads, dim] per layer")
        return cls(layers, block_tokens, h, d, slots // block_tokens,
                   block_stride=block_tokens * 2 * h * d, kv_stride=h * d, token_stride=2 * h * d)

    @classmethod
    def from_block_kv_layers(cls, layers: Sequence[torch.Tensor]):
        """layers[l] is [blocks, 2, block_tokens, heads, dim] (Bi-KV/Model/qwen2.py:532-536)."""
        blocks, two, p, h, d = layers[0].shape
        if two != 2:
            raise RuntimeError("expected [blocks, 2, block_tokens, heads, dim] per layer")
        return cls(layers, p, h, d, blocks, block_stride=2 * p * h * d, kv_stride=p * h * d, token_stride=h * d)

    def page_list(self, block_ids, tm_pages=None, sort: bool = False, check_unique: bool = False):
        """Uploads a page list built on the host (where a block manager keeps its lists): returns the
        device tensors (block_ids, tm_pages) to pass to load_token_major / store_token_major, in one
        upload. With `sort` the pages are reordered by ascending block id — the result is the same, the
        order in which the kernel walks the pool is not: neighbouring workgroups then touch neighbouring
        blocks of every layer tensor while the token-major pages are visited in a scattered order.
        Measured on MI355X at the reference's shape (4096 of 10240 blocks) with a torch-allocated pool
        that sits in one half of HBM: a LOAD gains ~4 % (its scattered side is the written one), a STORE
        loses ~7 % (its dense writes become scattered). On a pool from bikv_device_alloc, whose chunks
        alternate between the halves, the order makes no difference. `tm_pages` defaults to 0..n-1
        BEFORE sorting, i.e. page i of the token-major buffer belongs to block_ids[i]."""
        import numpy as np
        ids = np.ascontiguousarray(np.asarray(block_ids, dtype=np.int64).reshape(-1))
        tm = (np.arange(ids.size, dtype=np.int64) if tm_pages is None
              else np.ascontiguousarray(np.asarray(tm_pages, dtype=np.int64).reshape(-1)))
        if tm.size != ids.size:
            raise RuntimeError("block_ids and tm_pages differ in length")
        if check_unique:
            _lib.require_unique(ids, "block ids")
        if sort and ids.size > 1:
            order = np.argsort(ids, kind="stable")
            ids, tm = ids[order], tm[order]
        both = torch.from_numpy(np.stack([ids, tm])).to(self.device)     # one upload
        return both[0], both[1]

    def _call(self, fn, tm: torch.Tensor, block_ids: torch.Tensor, tm_pages: Optional[torch.Tensor]):
        if not tm.is_contiguous() or not (tm.is_cuda or tm.is_pinned()):
            # pinned host memory is mapped into the device's address space: the kernel reads / writes it over
            # the host link, which is how a transport's host region is filled or drained without a hop
            raise RuntimeError("token-major buffer must be a contiguous CUDA tensor or pinned host memory")
        if tm.element_size() != self._layers[0].element_size():
            raise RuntimeError("token-major buffer and pool differ in element size")
        if tm_pages is None:
            tm_pages = torch.arange(block_ids.numel(), dtype=torch.int64, device=self.device)
        for name, t in (("block_ids", block_ids), ("tm_pages", tm_pages)):
            if not t.is_cuda or t.dtype != torch.int64 or t.dim() != 1 or not t.is_contiguous():
                raise RuntimeError(f"{name} must be a contiguous 1-D int64 CUDA tensor")
        if tm_pages.numel() != block_ids.numel():
            raise RuntimeError("block_ids and tm_pages differ in length")
        with torch.cuda.device(self.device):
            _lib.check(fn(self._h, tm.data_ptr(), tm.numel() * tm.element_size(), block_ids.data_ptr(),
                          tm_pages.data_ptr(), block_ids.numel(),
                          C.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)))

    def load_token_major(self, tm: torch.Tensor, block_ids: torch.Tensor, tm_pages: Optional[torch.Tensor] = None,
                         check_unique: bool = False):
        """Received token-major pages -> pool blocks (unique block ids). `tm` holds pages of
        block_tokens tokens, each token [dim][heads][layers][2]; page i of the call is tm page
        tm_pages[i] (default: i). Asynchronous on the current stream. `check_unique=True` copies the
        block ids to the host first (a synchronising debug aid) and raises RuntimeError naming the first
        block that is named twice."""
        if check_unique:
            _lib.require_unique(block_ids.cpu().numpy(), "load_token_major block ids")
        self._call(_lib.load().bikv_nhd_load_token_major, tm, block_ids, tm_pages)

    def store_token_major(self, tm: torch.Tensor, block_ids: torch.Tensor, tm_pages: Optional[torch.Tensor] = None):
        """Pool blocks -> token-major pages (unique tm pages). Asynchronous on the current stream."""
        self._call(_lib.load().bikv_nhd_store_token_major, tm, block_ids, tm_pages)

    def check(self):
        idx = self.device.index if self.device.index is not None else torch.cuda.current_device()
        with torch.cuda.device(self.device):
            _lib.check(_lib.load().bikv_check_status(
                idx, C.c_void_p(torch.cuda.current_stream(self.device).cuda_stream), None))

    def close(self):
        if getattr(self, "_h", None):
            _lib.load().bikv_nhd_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
