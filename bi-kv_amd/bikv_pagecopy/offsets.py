"""Offset tables for the run copy, built from the coordinator's page lists.

Mirror of the index stage of KVCache.shared_data_batch_pages
(Bi-KV/DistributedStorage/kvcache.py:161-196): `cache_pages_list[k]` holds the page ids of item k
and `id_token_pair[k][1]` its token count; every page becomes one run whose source offset is
`page * page_size` and whose destination offset is the running sum of the page sizes, where the
last page of an item counts only `tokens % page_size` tokens when that is non-zero.

The reference computes these offsets in TOKENS and hands them to a kernel that reads them as
ELEMENTS (copy_kernel.cu:22-33), so as shipped it copies from the wrong place; the two reference
scripts that exercise the kernel pass element offsets (test_page_ipc.py:58-65). `unit="elements"`
(default) multiplies by elements_per_token and is what a correct caller needs; `unit="tokens"`
reproduces the reference's literal numbers.

The reference builds the lists with two nested Python loops and two `torch.tensor(list)` uploads;
this builder is vectorised numpy and produces one [2, n] array for a single upload.
"""
from typing import Sequence, Tuple

import numpy as np
import torch


def build_run_offsets(cache_pages_list: Sequence[Sequence[int]], item_tokens: Sequence[int],
                      page_size: int, elements_per_token: int = 1,
                      unit: str = "elements", with_sizes: bool = False) -> Tuple[np.ndarray, int]:
    """Returns (offsets, total_tokens): offsets[0] = source offsets, offsets[1] = destination offsets,
    both int64, one entry per page in list order; total_tokens = sum of the copied page sizes.
    with_sizes=True adds a third row, the tokens each run holds (page_size, or the tail of an item's
    partial last page): the run lengths a packed destination needs (always in tokens)."""
    if unit not in ("elements", "tokens"):
        raise ValueError("unit must be 'elements' or 'tokens'")
    if page_size <= 0:
        raise ValueError("page_size must be positive")
    if len(cache_pages_list) != len(item_tokens):
        raise ValueError("cache_pages_list and item_tokens differ in length")
    counts = np.fromiter((len(p) for p in cache_pages_list), dtype=np.int64, count=len(cache_pages_list))
    n = int(counts.sum())
    out = np.empty((3 if with_sizes else 2, n), dtype=np.int64)
    if n == 0:
        return out, 0
    pages = np.concatenate([np.asarray(p, dtype=np.int64).reshape(-1) for p in cache_pages_list if len(p)])
    tokens = np.asarray(item_tokens, dtype=np.int64)
    sizes = np.full(n, page_size, dtype=np.int64)
    last = np.cumsum(counts) - 1                      # index of each item's last page
    has = counts > 0
    tail = tokens % page_size
    partial = has & (tail != 0)
    sizes[last[partial]] = tail[partial]
    dst = np.zeros(n, dtype=np.int64)
    np.cumsum(sizes[:-1], out=dst[1:])
    scale = elements_per_token if unit == "elements" else 1
    out[0] = pages * page_size * scale
    out[1] = dst * scale
    if with_sizes:
        out[2] = sizes
    return out, int(sizes.sum())


class RunIndexPool:
    """Persistent device index buffers, as KVCache keeps them (kvcache.py:60-64, `src_index_pool` /
    `dst_index_pool` of `max_pages` int64 entries each, handed out by `get_index_tensors`, :83-86 —
    which returns the source pool twice; here the rows are distinct). One device tensor of `rows` x
    `max_pages` int64 and a pinned host mirror: `load()` copies a freshly built offset table into the
    mirror and uploads it with one asynchronous copy on the current stream, so a transfer allocates
    nothing and never uploads from pageable memory."""

    def __init__(self, max_pages: int, device, rows: int = 3):
        self.max_pages = int(max_pages)
        self.rows = int(rows)
        self.device = torch.device(device)
        self.dev = torch.full((self.rows * self.max_pages,), -1, dtype=torch.int64, device=self.device)
        self.host = torch.empty(self.rows * self.max_pages, dtype=torch.int64, pin_memory=True)
        self._host_np = self.host.numpy()
        self._busy = None

    def load(self, table: np.ndarray) -> torch.Tensor:
        """table: [r, n] int64 with r <= rows, n <= max_pages. Returns it as an [r, n] device tensor
        (the leading r*n entries of the buffer), valid until the next load()."""
        r, n = table.shape
        if r > self.rows or n > self.max_pages:
            raise RuntimeError(f"Requested {n} exceeds pool size {self.max_pages}")   # kvcache.py:84
        if self._busy is not None:
            self._busy.synchronize()          # the previous upload still reads the mirror
        self._host_np[: r * n].reshape(r, n)[...] = table
        self.dev[: r * n].copy_(self.host[: r * n], non_blocking=True)
        if self._busy is None:
            self._busy = torch.cuda.Event()
        self._busy.record(torch.cuda.current_stream(self.device))
        return self.dev[: r * n].view(r, n)
