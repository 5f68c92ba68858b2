"""Pins the CPU oracle before anything is compared against it.

Checks, chosen so that a plausible mistake fails at least one of them:
  * the two known-answer scenarios the reference's own scripts hold (shape bookkeeping, value 7);
  * the library routines the formula reduces to (numpy fancy indexing, torch.index_select /
    index_copy_) — a swapped src/dst offset, a wrong unit or a transposed slot order fails here;
  * per-byte brute force on tiny inputs;
  * invariants: permutation round trip, duplicate ids -> identical rows, order of ids = order of rows,
    bytes outside the written runs untouched (0xA5 canaries);
  * the committed config-1 digests.
"""
import hashlib
import json
import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


@pytest.fixture(scope="module")
def scenarios():
    with open(os.path.join(GOLDEN, "reference_scenarios.json")) as f:
        return json.load(f)


# ---- the reference's own known answers ---------------------------------------------------------
def test_reference_page_ipc_scenario(oracle, scenarios):
    s = scenarios["test_page_ipc"]
    ept = s["head_size"] * s["num_kv_heads"] * s["num_layers"] * s["kv_pair"]
    page_elements = s["page_size"] * ept
    assert page_elements == 716800  # "716800 elements/page", test_page_ipc.py:43
    n = s["num_pages"]
    cache = np.full(n * page_elements, s["fill_value"], dtype=np.float16)
    ring = oracle.Ring(buffer_size=s["buffer_size"])
    offs = np.arange(n, dtype=np.int64) * page_elements
    dims = (s["head_size"], s["num_kv_heads"], s["num_layers"], s["kv_pair"])
    buf = np.zeros(2 * n * page_elements, dtype=np.float16)  # room for two transfers
    for k in range(2):
        at = oracle.ring_step_c(ring, n, s["page_size"], dims, 2)
        assert at == k * n * page_elements * 2
        window = buf[at // 2:]
        assert oracle.copy_runs_c(cache, window, offs, offs, page_elements) == 0
        assert ring.tensor_dim == s["expected_dim"]
        assert list(ring.tensor_shape) == s["expected_shape"]
        assert ring.last_valid_offset == at
        got = buf[at // 2: at // 2 + n * page_elements].reshape(s["expected_shape"])
        assert np.all(got == s["expected_value"])


def test_reference_zero_copy_scenario(oracle, scenarios):
    s = scenarios["test_zero_copy"]
    ept = s["head_size"] * s["num_kv_heads"] * s["num_layers"] * s["kv_pair"]
    page_elements = s["page_size"] * ept
    n = s["num_pages"]
    cpu = np.full(n * page_elements, s["fill_value"], dtype=np.float16)
    page_indices = np.arange(n, dtype=np.int64)          # element offsets, unscaled
    dest = np.arange(0, n * page_elements, page_elements, dtype=np.int64)
    out = np.zeros(n * page_elements, dtype=np.float16)
    assert oracle.copy_runs_c(cpu, out, page_indices, dest, page_elements) == 0
    assert np.all(out.reshape(s["expected_shape"]) == s["expected_value"])
    # that the indices really are element offsets shows on non-constant data
    ramp = (np.arange(4096) % 251).astype(np.float16)
    out2 = np.zeros(3 * 16, dtype=np.float16)
    oracle.copy_runs_c(ramp, out2, [0, 1, 2], [0, 16, 32], 16)
    assert np.array_equal(out2.reshape(3, 16)[1], ramp[1:17])


# ---- run copy vs library routine and brute force ---------------------------------------------
@pytest.mark.parametrize("dtype", [np.uint8, np.float16, np.float32, np.float64])
def test_copy_runs_three_statements_agree(oracle, dtype):
    rng = np.random.default_rng(11)
    run = 24
    src = rng.integers(0, 255, size=40 * run * np.dtype(dtype).itemsize, dtype=np.uint8).view(dtype)
    n = 17
    so = rng.integers(0, src.size - run, size=n)             # overlapping / repeated sources are legal
    do = rng.permutation(60)[:n] * run                       # disjoint destinations
    outs = []
    for fn in (oracle.copy_runs_c, oracle.copy_runs_np, oracle.copy_runs_loops):
        dst = np.full(60 * run, 0, dtype=dtype)
        dst.view(np.uint8)[:] = 0xA5
        fn(src, dst, so, do, run)
        outs.append(dst.tobytes())
    assert outs[0] == outs[1] == outs[2]
    # canaries: every run not targeted still holds 0xA5
    dst = np.frombuffer(outs[0], dtype=np.uint8).reshape(60, -1)
    untouched = np.setdiff1d(np.arange(60), do // run)
    assert np.all(dst[untouched] == 0xA5)
    assert not np.all(dst[do // run] == 0xA5)


def test_copy_runs_equals_index_select_and_index_copy(oracle):
    rng = np.random.default_rng(5)
    pages, page_elems = 64, 96
    pool = rng.standard_normal((pages, page_elems)).astype(np.float16)
    ids = rng.permutation(pages)[:20]
    dense = np.arange(20, dtype=np.int64) * page_elems
    # gather: scattered source offsets, dense destinations == index_select
    out = np.zeros((20, page_elems), dtype=np.float16)
    oracle.copy_runs_c(pool, out, ids * page_elems, dense, page_elems)
    want = torch.index_select(torch.from_numpy(pool), 0, torch.from_numpy(ids)).numpy()
    assert out.tobytes() == want.tobytes()
    # scatter: the same call with the roles swapped == index_copy_
    ids2 = rng.permutation(pages)[:20]
    pool2 = pool.copy()
    oracle.copy_runs_c(out, pool2, dense, ids2 * page_elems, page_elems)
    want2 = torch.from_numpy(pool.copy()).index_copy_(0, torch.from_numpy(ids2), torch.from_numpy(out)).numpy()
    assert pool2.tobytes() == want2.tobytes()


def test_copy_runs_skips_out_of_range(oracle):
    src = np.arange(100, dtype=np.uint8)
    dst = np.zeros(100, dtype=np.uint8)
    skipped = oracle.copy_runs_c(src, dst, [0, 95, -1, 10], [0, 10, 20, 96], 10)
    assert skipped == 3
    assert np.array_equal(dst[:10], src[:10]) and not dst[10:].any()


# ---- ring bookkeeping ---------------------------------------------------------------------------
def test_ring_step_wraps_like_the_reference(oracle):
    dims = (128, 2, 28, 2)
    per = 3 * 50 * 14336 * 2
    ring = oracle.Ring(buffer_size=int(2.5 * per))
    state = {"current_offset": 0, "last_valid_offset": 0, "buffer_size": int(2.5 * per)}
    seen = []
    for _ in range(5):
        a = oracle.ring_step_c(ring, 3, 50, dims, 2)
        b = oracle.ring_step_py(state, 3, 50, dims, 2)
        assert a == b == ring.last_valid_offset == state["last_valid_offset"]
        assert ring.current_offset == state["current_offset"] == a + per
        assert list(ring.tensor_shape) == state["tensor_shape"] == [150, 128, 2, 28, 2]
        assert ring.data_size == per
        seen.append(a)
    assert seen == [0, per, 0, per, 0]  # third batch does not fit behind 2*per -> restart at 0


def test_ring_send_publishes_real_shape(oracle):
    ring = oracle.Ring(buffer_size=1000)
    assert oracle.ring_send_c(ring, 600, [10, 30]) == 0
    assert (ring.tensor_dim, list(ring.tensor_shape)[:2], ring.data_size) == (2, [10, 30], 600)
    assert oracle.ring_send_c(ring, 600, [5, 6, 10]) == 0  # 600+600 > 1000 -> wrap
    assert ring.last_valid_offset == 0 and ring.current_offset == 600 and ring.tensor_dim == 3
    assert oracle.ring_send_c(ring, 300, [150]) == 600


# ---- offset tables ------------------------------------------------------------------------------
def test_build_offsets_matches_reference_loops(oracle):
    rng = np.random.default_rng(3)
    page_size = 16
    for _ in range(50):
        n_items = int(rng.integers(0, 6))
        tokens = rng.integers(1, 100, size=n_items)
        lists = [rng.permutation(1000)[: -(-int(t) // page_size)].tolist() for t in tokens]
        pairs = [(k, int(t)) for k, t in enumerate(tokens)]
        for scale in (1, 14336):
            so, do, total = oracle.build_offsets_loops(lists, pairs, page_size, scale)
            so_c, do_c, total_c = oracle.build_offsets_c(lists, tokens, page_size, scale)
            assert so == so_c.tolist() and do == do_c.tolist() and total == total_c
            assert total == int(tokens.sum())  # partial last pages count their real tokens


def test_build_offsets_hand_example(oracle):
    # two items: 40 tokens on pages [7, 2, 9] (16-token pages -> sizes 16, 16, 8), 16 tokens on [4]
    so, do, total = oracle.build_offsets_loops([[7, 2, 9], [4]], [(0, 40), (1, 16)], 16)
    assert so == [112, 32, 144, 64]
    assert do == [0, 16, 32, 40]
    assert total == 56


# ---- layered gather / scatter -----------------------------------------------------------------
@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
def test_layered_statements_agree(oracle, layout):
    rng = np.random.default_rng(8)
    pool = rng.integers(0, 2 ** 16, size=(6, 40, 8), dtype=np.uint16)
    reqs = [rng.permutation(40)[:5], np.array([3, 3, 7], dtype=np.int64), np.zeros(0, dtype=np.int64),
            rng.permutation(40)[:1]]
    a = oracle.gather_layered_c(pool, reqs, layout)
    b = oracle.gather_layered_np(pool, reqs, layout)
    c = oracle.gather_layered_loops(pool, reqs, layout)
    assert a.tobytes() == b.tobytes() == c.tobytes()
    # the slot formula, spelled out for one element
    m0 = 5
    q, j = 4, 2
    slot = q * m0 + j if layout == "layer_major" else j * 6 + q
    assert np.array_equal(a.reshape(-1, 8)[slot], pool[q, reqs[0][j]])
    # duplicates give identical rows; order of ids is order of rows
    second = a.reshape(-1, 8)[m0 * 6:]
    if layout == "layer_major":
        r = second[: 3 * 6].reshape(6, 3, 8)
        assert np.array_equal(r[:, 0], r[:, 1]) and np.array_equal(r[:, 2], pool[:, 7])
    else:
        r = second[: 3 * 6].reshape(3, 6, 8)
        assert np.array_equal(r[0], r[1]) and np.array_equal(r[2], pool[:, 7])


@pytest.mark.parametrize("layout", ["layer_major", "page_major"])
def test_layered_scatter_inverts_gather(oracle, layout):
    rng = np.random.default_rng(9)
    pool = rng.integers(0, 255, size=(4, 32, 16), dtype=np.uint8)
    perm = rng.permutation(32)
    reqs = [perm[:10], perm[10:11], perm[11:32]]
    staged = oracle.gather_layered_c(pool, reqs, layout)
    for scatter in (oracle.scatter_layered_c, oracle.scatter_layered_np):
        blank = np.full_like(pool, 0xA5)
        scatter(blank, reqs, staged, layout)
        assert blank.tobytes() == pool.tobytes()  # a permutation round trip is the identity
    # partial scatter leaves the other pages untouched
    blank = np.full_like(pool, 0xA5)
    oracle.scatter_layered_c(blank, [perm[:10]], oracle.gather_layered_c(pool, [perm[:10]], layout), layout)
    assert np.array_equal(blank[:, perm[:10]], pool[:, perm[:10]])
    assert np.all(blank[:, perm[10:]] == 0xA5)


def test_layered_equals_torch_cpu_path(oracle):
    rng = np.random.default_rng(10)
    pool = rng.standard_normal((4, 50, 32)).astype(np.float16)
    ids = rng.permutation(50)[:12]
    got = oracle.gather_layered_c(pool, [ids]).reshape(4, 12, 32)
    want = oracle.gather_layered_torch(torch.from_numpy(pool), torch.from_numpy(ids)).numpy()
    assert got.tobytes() == want.tobytes()
    ids2 = rng.permutation(50)[:12]
    p_c = pool.copy()
    oracle.scatter_layered_c(p_c, [ids2], got.reshape(-1))
    p_t = torch.from_numpy(pool.copy())
    oracle.scatter_layered_torch(p_t, torch.from_numpy(ids2), torch.from_numpy(got))
    assert p_c.tobytes() == p_t.numpy().tobytes()


def test_config1_golden_digests(oracle):
    from bikv_pagecopy import workloads
    with open(os.path.join(GOLDEN, "config1.json")) as f:
        g = json.load(f)
    shape = workloads.SHAPES["tiny"]
    pool = np.random.default_rng(0).standard_normal(
        (shape.n_planes, shape.n_pages, shape.tile_bytes // 2)).astype(np.float16)
    assert _sha(pool) == g["pool_sha256"]
    wl = workloads.named("tiny")
    assert wl["gather"][0].tolist() == g["gather_ids"] and wl["scatter"][0].tolist() == g["scatter_ids"]
    for layout in ("layer_major", "page_major"):
        st = oracle.gather_layered_c(pool, wl["gather"], layout)
        assert _sha(st) == g[layout]["staging_sha256"]
        p = pool.copy()
        oracle.scatter_layered_c(p, wl["scatter"], st, layout)
        assert _sha(p) == g[layout]["pool_after_scatter_sha256"]


# ---- fused page move + layout change -----------------------------------------------------------
@pytest.mark.parametrize("form", ["token_kv", "block_kv"])
@pytest.mark.parametrize("dtype", [np.uint8, np.uint16, np.uint32])
def test_transpose_pages_statements_agree(oracle, form, dtype):
    rng = np.random.default_rng(14)
    P, D, H, L, blocks, n_tm = 4, 8, 2, 3, 7, 5
    tm = rng.integers(0, np.iinfo(dtype).max, size=(n_tm, P, D, H, L, 2), dtype=dtype)
    shape = (blocks * P, 2, H, D) if form == "token_kv" else (blocks, 2, P, H, D)
    block_ids, tm_pages = np.array([5, 0, 3]), np.array([4, 1, 2])
    la = [np.zeros(shape, dtype=dtype) for _ in range(L)]
    for a in la:
        a.view(np.uint8)[...] = 0xA5
    lb = [a.copy() for a in la]
    assert oracle.transpose_pages_c(la, form, tm, block_ids, tm_pages, "load") == 0
    oracle.transpose_pages_np(lb, form, tm, block_ids, tm_pages, "load")
    for a, b in zip(la, lb):
        assert a.tobytes() == b.tobytes()
    # one element by hand: page 0 of the call (block 5, tm page 4), token 2, d 6, head 1, layer 2, V
    want = tm[4, 2, 6, 1, 2, 1]
    got = la[2][5 * P + 2, 1, 1, 6] if form == "token_kv" else la[2][5, 1, 2, 1, 6]
    assert got == want
    # blocks that were not named keep their canary
    untouched = la[0][1 * P:(1 + 1) * P] if form == "token_kv" else la[0][1]
    assert np.all(untouched.view(np.uint8) == 0xA5)
    # store is the inverse of load
    tm2 = np.zeros_like(tm)
    tm3 = np.zeros_like(tm)
    assert oracle.transpose_pages_c(la, form, tm2, block_ids, tm_pages, "store") == 0
    oracle.transpose_pages_np(la, form, tm3, block_ids, tm_pages, "store")
    assert tm2.tobytes() == tm3.tobytes()
    assert np.array_equal(tm2[tm_pages], tm[tm_pages]) and not tm2[[0, 3]].any()
    # out-of-range ids are skipped and counted
    assert oracle.transpose_pages_c(la, form, tm, np.array([7, 1]), np.array([0, 9]), "load") == 2


def test_transpose_pages_equals_the_flat_token_major_formula(oracle):
    """The token-major page really is the reference's (tokens,)+token_shape buffer: flat element
    offset (((t*D + d)*H + h)*L + l)*2 + k with token_shape = (D, H, L, 2)."""
    P, D, H, L = 2, 8, 2, 4
    tm = np.arange(1 * P * D * H * L * 2, dtype=np.uint16).reshape(1, P, D, H, L, 2)
    layers = [np.zeros((3 * P, 2, H, D), dtype=np.uint16) for _ in range(L)]
    oracle.transpose_pages_c(layers, "token_kv", tm, [2], [0], "load")
    t, d, h, l, k = 1, 5, 1, 3, 0
    assert layers[l][2 * P + t, k, h, d] == (((t * D + d) * H + h) * L + l) * 2 + k


# ---- ragged runs (packed destinations of partial last pages) -----------------------------------
def test_ragged_copy_reduces_to_the_uniform_copy_and_to_brute_force(oracle):
    rng = np.random.default_rng(51)
    src = rng.integers(0, 65536, size=4000, dtype=np.uint16)
    n, run = 23, 96
    so = rng.integers(0, 4000 - run, size=n)
    do = rng.permutation(n) * run
    a = np.full(n * run, 0xA5A5, dtype=np.uint16)
    b = a.copy()
    assert oracle.copy_runs_ragged_c(src, a, so, do, np.full(n, run), run) == 0
    assert oracle.copy_runs_c(src, b, so, do, run) == 0
    assert a.tobytes() == b.tobytes()                      # all lengths equal -> the uniform copy
    lens = rng.integers(0, run + 1, size=n)
    lens[:2] = (0, run)
    c = np.full(n * run, 0xA5A5, dtype=np.uint16)
    assert oracle.copy_runs_ragged_c(src, c, so, do, lens, run) == 0
    want = np.full(n * run, 0xA5A5, dtype=np.uint16)
    for p in range(n):                                      # brute force, element by element
        for e in range(int(lens[p])):
            want[do[p] + e] = src[so[p] + e]
    assert c.tobytes() == want.tobytes()
    # units: offsets and lengths in blocks of 8 elements
    d = np.full(n * run, 0xA5A5, dtype=np.uint16)
    lens8 = rng.integers(0, run // 8 + 1, size=n)
    so8 = rng.integers(0, (4000 - run) // 8, size=n)
    do8 = rng.permutation(n) * (run // 8)
    assert oracle.copy_runs_ragged_c(src, d, so8, do8, lens8, run // 8, unit_elems=8) == 0
    want = np.full(n * run, 0xA5A5, dtype=np.uint16)
    for p in range(n):
        want[do8[p] * 8: do8[p] * 8 + lens8[p] * 8] = src[so8[p] * 8: so8[p] * 8 + lens8[p] * 8]
    assert d.tobytes() == want.tobytes()


def test_ragged_copy_skips_bad_lengths_and_ranges(oracle):
    src = np.arange(100, dtype=np.uint16)
    dst = np.zeros(100, dtype=np.uint16)
    so = np.array([0, 10, 20, 95, 40])
    do = np.array([0, 10, 20, 30, 96])
    lens = np.array([5, -1, 11, 6, 5])                      # ok, negative, above max, src overrun, dst overrun
    assert oracle.copy_runs_ragged_c(src, dst, so, do, lens, 10) == 4
    assert dst[:5].tolist() == [0, 1, 2, 3, 4] and not dst[5:].any()


def test_packed_offsets_with_tail_lengths_deliver_exactly_each_items_tokens(oracle):
    """The reference's packed destination offsets (kvcache.py:161-174), restated by build_offsets_loops,
    are consistent with ONE thing only: copying `tail` tokens of a partial last page. Stated without
    any offsets, the transfer is 'each item's rows, cut to its token count, back to back'."""
    rng = np.random.default_rng(52)
    page_size, ept, pool_pages = 16, 12, 40
    pool = rng.integers(0, 65536, size=(pool_pages * page_size, ept), dtype=np.uint16)
    pages_list = [[7, 2, 39], [4], [], [30, 31, 0], [5, 6]]
    tokens = [40, 16, 0, 33, 17]
    so, do, total = oracle.build_offsets_loops(pages_list, [(0, t) for t in tokens], page_size)   # token units
    sizes = []
    for pages, t in zip(pages_list, tokens):
        sizes += [page_size] * (len(pages) - 1) + ([t % page_size or page_size] if pages else [])
    assert total == sum(sizes) == 40 + 16 + 33 + 17
    dst = np.full((total, ept), 0xA5A5, dtype=np.uint16)
    assert oracle.copy_runs_ragged_c(pool, dst, so, do, sizes, page_size, unit_elems=ept) == 0
    want = oracle.packed_items_np(pool, pages_list, tokens, page_size)
    assert want.shape == dst.shape and dst.tobytes() == want.tobytes()
    # whole-page copies into the same packed offsets write past an item's end: the last run alone
    # already leaves the buffer
    over = np.full((total, ept), 0xA5A5, dtype=np.uint16)
    assert oracle.copy_runs_c(pool, over, np.asarray(so) * ept, np.asarray(do) * ept, page_size * ept) >= 1


def test_worker_form_planes_are_the_tokens_of_each_block(oracle):
    """planes_of_token_kv_layers against explicit indexing: element (plane 2l+k, block b, token t, head h, d)
    is layers[l][b*P + t, k, h, d]; and the inverse restores the layers."""
    rng = np.random.default_rng(71)
    P, H, D, L, blocks = 4, 3, 8, 2, 5
    layers = [rng.integers(0, 65536, size=(blocks * P, 2, H, D), dtype=np.uint16) for _ in range(L)]
    planes = oracle.planes_of_token_kv_layers(layers, P)
    assert planes.shape == (2 * L, blocks, P * H * D)
    for l in range(L):
        for k in (0, 1):
            for b in range(blocks):
                for t in range(P):
                    got = planes[2 * l + k, b].reshape(P, H, D)[t]
                    assert np.array_equal(got, layers[l][b * P + t, k])
    back = oracle.token_kv_layers_of_planes(planes, P, H, D)
    assert all(np.array_equal(a, b) for a, b in zip(back, layers))


def _golden_cases():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(GOLDEN, "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_packed_transfer_and_layout_change_golden_digests(oracle):
    mg = _golden_cases()
    with open(os.path.join(GOLDEN, "packed_and_layout.json")) as f:
        g = json.load(f)
    pool, pages_list, tokens, page_size = mg.packed_case()
    assert _sha(pool) == g["packed_transfer"]["pool_sha256"]
    want = oracle.packed_items_np(pool, pages_list, tokens, page_size)
    assert want.shape[0] == g["packed_transfer"]["total_tokens"] and _sha(want) == g["packed_transfer"]["received_sha256"]
    for form in ("token_kv", "block_kv"):
        tm, layers, load, store = mg.layout_case(form)
        e = g[f"layout_change_{form}"]
        assert _sha(tm) == e["tm_sha256"] and _sha(np.stack(layers)) == e["layers_sha256"]
        assert oracle.transpose_pages_c(layers, form, tm, load[0], load[1], "load") == 0
        assert _sha(np.stack(layers)) == e["layers_after_load_sha256"]
        assert oracle.transpose_pages_c(layers, form, tm, store[0], store[1], "store") == 0
        assert _sha(tm) == e["tm_after_store_sha256"]
