"""The Worker-side callers (bikv_pagecopy/worker_calls.py, mirrors of Bi-KV/Worker/Worker.py:162-218) on a real
GPU: received KV lands in the Worker's per-layer paged cache, outgoing KV leaves it, through the ring (same
box) and through a pinned host image (other box), whole and partly filled last blocks. Expected bytes come
from the oracle's layout change."""
import os
from types import SimpleNamespace

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

D, H, L, P = 64, 2, 4, 16                      # token_shape (D, H, L, 2); blocks (and cache pages) of 16 tokens
DIMS = (D, H, L, 2)


@pytest.fixture()
def ring(lib, cuda):
    import ipc_service
    ipc_service.producer_cleanup()
    ipc_service.consumer_cleanup()
    name = f"/bikv_test_worker_{os.getpid()}"
    ipc_service.consumer_init(0, name, 32 << 20)
    ipc_service.producer_init(0, name)
    yield ipc_service
    ipc_service.producer_cleanup()
    ipc_service.consumer_cleanup()


def _worker_cache(cuda, rng, blocks=24):
    import bikv_pagecopy as bk
    layers_h = [rng.integers(0, 65536, size=(blocks * P, 2, H, D), dtype=np.uint16) for _ in range(L)]
    layers_d = [torch.from_numpy(a.view(np.int16)).view(torch.float16).to(cuda) for a in layers_h]
    return layers_h, layers_d, bk.NHDPool.from_token_kv_layers(layers_d, P)


def _same(layers_d, layers_h):
    return all(layers_d[l].cpu().view(torch.int16).numpy().tobytes() == layers_h[l].tobytes() for l in range(L))


def _pages_of(tokens_h, n_tokens):
    """A token-major image [tokens, ...] cut into pages of P tokens, the last one padded with zeros."""
    n = -(-n_tokens // P)
    out = np.zeros((n, P) + DIMS, dtype=np.uint16)
    out.reshape((n * P,) + DIMS)[:n_tokens] = tokens_h[:n_tokens]
    return out


@pytest.mark.parametrize("as_dict", [False, True])
def test_received_kv_from_the_ring_lands_in_the_paged_cache(ring, oracle, cuda, as_dict):
    """Cache side -> ring -> Worker, both through the mirrors of the reference's methods; the coordinator's
    message as a protobuf-like object and as a dict."""
    from bikv_pagecopy import kvcache_calls, worker_calls
    print(f"[case] worker receive through the ring (dict={as_dict})", flush=True)
    rng = np.random.default_rng(601)
    cache_pages = 40
    cache_h = rng.integers(0, 65536, size=(cache_pages * P,) + DIMS, dtype=np.uint16)
    cache_d = torch.from_numpy(cache_h.view(np.int16)).view(torch.float16).to(cuda)
    layers_h, layers_d, kv = _worker_cache(cuda, rng)
    pages_list = [[31, 4, 17], [9, 38]]
    fields = {"infer_worker": 0, "cache_worker": 0, "token_num": 5 * P,
              "id_token_pair": [(100, 3 * P), (101, 2 * P)], "cache_pages_list": pages_list}
    kvcache_calls.shared_data_batch_pages(cache_d, fields, P, DIMS)
    info = fields if as_dict else SimpleNamespace(**fields)
    blocks = [20, 3, 11, 7, 0]
    assert worker_calls.receive_kvcache_data_batch(info, kv, blocks, worker_index=0, timeout_ms=5000) == 5 * P
    flat = [p for pages in pages_list for p in pages]
    tm_h = np.stack([cache_h[p * P:(p + 1) * P] for p in flat])
    assert oracle.transpose_pages_c(layers_h, "token_kv", tm_h, np.array(blocks), np.arange(5), "load") == 0
    assert _same(layers_d, layers_h)
    t = worker_calls.last_stage_times()
    assert (t.tokens, t.pages) == (5 * P, 5) and t.total_ms >= t.layout_ms > 0
    kv.close()


def test_a_partly_filled_last_block_is_received_token_exact(ring, oracle, cuda):
    """2 blocks and 5 tokens: the packed transfer of the cache side publishes exactly that many tokens, the
    Worker writes two whole blocks and a third whose remaining slots become zeros."""
    from bikv_pagecopy import kvcache_calls, worker_calls
    print("[case] worker receive, partial last block", flush=True)
    rng = np.random.default_rng(603)
    cache_h = rng.integers(0, 65536, size=(30 * P,) + DIMS, dtype=np.uint16)
    cache_d = torch.from_numpy(cache_h.view(np.int16)).view(torch.float16).to(cuda)
    layers_h, layers_d, kv = _worker_cache(cuda, rng)
    n_tok = 2 * P + 5
    fields = {"infer_worker": 0, "cache_worker": 0, "token_num": n_tok, "id_token_pair": [(7, n_tok)],
              "cache_pages_list": [[12, 3, 25]]}
    _, published = kvcache_calls.shared_data_batch_pages(cache_d, fields, P, DIMS, pack_partial_pages="exact")
    assert published == n_tok
    blocks = [9, 1, 16]
    worker_calls.receive_kvcache_data_batch(SimpleNamespace(**fields), kv, blocks, worker_index=0, timeout_ms=5000)
    tokens_h = np.concatenate([cache_h[12 * P:13 * P], cache_h[3 * P:4 * P], cache_h[25 * P:25 * P + 5]])
    tm_h = _pages_of(tokens_h, n_tok)
    assert oracle.transpose_pages_c(layers_h, "token_kv", tm_h, np.array(blocks), np.arange(3), "load") == 0
    assert _same(layers_d, layers_h)
    with pytest.raises(RuntimeError, match="block ids were given"):
        kvcache_calls.shared_data_batch_pages(cache_d, fields, P, DIMS, pack_partial_pages="exact")
        worker_calls.receive_kvcache_data_batch(SimpleNamespace(**fields), kv, [9, 1], worker_index=0, timeout_ms=5000)
    kv.close()


def test_kv_from_another_box_is_read_out_of_the_pinned_host_image(lib, oracle, cuda):
    from bikv_pagecopy import worker_calls
    import bikv_pagecopy as bk
    print("[case] worker receive from a pinned host image", flush=True)
    rng = np.random.default_rng(605)
    layers_h, layers_d, kv = _worker_cache(cuda, rng)
    n_tok = 3 * P + 9
    tokens_h = rng.integers(0, 65536, size=(n_tok,) + DIMS, dtype=np.uint16)
    host = bk.pinned_empty(n_tok * D * H * L * 2 * 2).view(torch.float16).view((n_tok,) + DIMS)
    host.view(torch.int16).copy_(torch.from_numpy(tokens_h.view(np.int16)))
    info = SimpleNamespace(cache_worker=3, token_num=n_tok, id_token_pair=[SimpleNamespace(id=1, token_num=n_tok)])
    blocks = [5, 22, 0, 13]
    assert worker_calls.receive_kvcache_data_batch(info, kv, blocks, worker_index=0, host_image=host) == n_tok
    tm_h = _pages_of(tokens_h, n_tok)
    assert oracle.transpose_pages_c(layers_h, "token_kv", tm_h, np.array(blocks), np.arange(4), "load") == 0
    assert _same(layers_d, layers_h)
    with pytest.raises(RuntimeError, match="pinned host image"):
        worker_calls.receive_kvcache_data_batch(info, kv, blocks, worker_index=0)
    with pytest.raises(RuntimeError, match="pinned"):
        worker_calls.receive_kvcache_data_batch(info, kv, blocks, worker_index=0, host_image=torch.zeros((n_tok,) + DIMS, dtype=torch.float16))
    kv.close()


def test_outgoing_kv_leaves_the_paged_cache_through_the_ring_and_through_a_host_image(ring, oracle, cuda):
    from bikv_pagecopy import worker_calls
    import bikv_pagecopy as bk
    print("[case] worker send", flush=True)
    rng = np.random.default_rng(607)
    layers_h, layers_d, kv = _worker_cache(cuda, rng)
    # the token count is the sum over id_token_pair (Worker.py:197-199): 2 blocks + 7 tokens
    pairs = [SimpleNamespace(id=4, token_num=P + 3), SimpleNamespace(id=9, token_num=P + 4)]
    total = 2 * P + 7
    blocks = [14, 2, 21]
    want = np.zeros((3, P) + DIMS, dtype=np.uint16)
    assert oracle.transpose_pages_c(layers_h, "token_kv", want, np.array(blocks), np.arange(3), "store") == 0
    want_tokens = want.reshape((3 * P,) + DIMS)[:total]
    # same box: through the ring
    info = SimpleNamespace(cache_worker=0, token_num=total, id_token_pair=pairs)
    assert worker_calls.send_kvcache_data_batch(info, kv, blocks, worker_index=0) == total
    got = ring.consumer_receive(timeout_ms=5000)
    assert tuple(got.shape) == (total,) + DIMS
    assert got.cpu().contiguous().view(torch.int16).numpy().tobytes() == want_tokens.tobytes()
    t = worker_calls.last_stage_times()
    assert (t.tokens, t.pages) == (total, 3) and t.publish_ms > 0
    # other box: straight into the transport's pinned region
    host = bk.pinned_empty(3 * P * D * H * L * 2 * 2).view(torch.float16)
    host.view(torch.int16).fill_(-1)
    info2 = {"cache_worker": 5, "token_num": total, "id_token_pair": [(4, P + 3), (9, P + 4)]}
    assert worker_calls.send_kvcache_data_batch(info2, kv, blocks, worker_index=0, host_image=host) == total
    assert host.view(torch.int16).numpy().tobytes() == want.tobytes()
    assert _same(layers_d, layers_h)                       # the cache itself is unchanged by sending
    with pytest.raises(RuntimeError, match="block ids were given"):
        worker_calls.send_kvcache_data_batch(info, kv, [1], worker_index=0)
    with pytest.raises(RuntimeError, match="pinned host image"):
        worker_calls.send_kvcache_data_batch(info2, kv, blocks, worker_index=0)
    kv.close()
