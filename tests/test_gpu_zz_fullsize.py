"""The four large configurations at their FULL pool sizes (30-137 GB resident in HBM), checked through
properties that do not need a CPU copy of the pool:

  * every gathered tile equals torch.index_select of its plane on the device (an independent
    implementation), for sampled planes of every request;
  * scatter into freshly allocated pages followed by a gather of those pages returns the scattered
    bytes exactly (round trip), for payload and scales;
  * pages that were not named keep their contents (plane checksums over the untouched pages);
  * requests sharing page ids (duplicates) produce identical rows.

The module name sorts last so that these allocations never coexist with another test's tensors.
"""
import gc

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _fill(t):
    flat = t.view(torch.uint8).reshape(-1)
    for off in range(0, flat.numel(), 1 << 31):
        flat[off: off + (1 << 31)].random_(0, 256)


def _cap(reqs, max_pages):
    out, used = [], 0
    for r in reqs:
        if out and used + len(r) > max_pages:
            break
        out.append(r)
        used += len(r)
    return out


def _check_against_index_select(pool_t, staging, batch, reqs, planes):
    for r, ids in enumerate(reqs):
        if len(ids) == 0:
            continue
        view = batch.request_view(staging, r)
        idt = torch.from_numpy(np.asarray(ids)).to(pool_t.device)
        for q in planes:
            got = view[q] if batch.layout == "layer_major" else view[:, q]
            assert torch.equal(got, torch.index_select(pool_t[q], 0, idt)), (r, q)


@pytest.mark.parametrize("name,layout", [
    ("qwen2_1p5b", "layer_major"), ("qwen2_7b", "layer_major"), ("qwen2_7b", "page_major"),
    ("llama3_8b", "layer_major"), ("llama3_70b_fp8", "page_major"), ("llama3_70b_fp8", "layer_major")])
def test_full_size_pool_properties(lib, cuda, name, layout):
    import bikv_pagecopy as bk
    from bikv_pagecopy import workloads as w
    shape = w.SHAPES[name]
    gc.collect()
    torch.cuda.empty_cache()          # hand the previous case's pool back to the driver
    free, _ = torch.cuda.mem_get_info(cuda)
    need = shape.pool_bytes + 3 * (16 << 30)
    if free < need:
        pytest.skip(f"needs {need / 1e9:.0f} GB of HBM, {free / 1e9:.0f} GB free")
    print(f"[case] full size {name} {layout}: pool {shape.pool_bytes / 1e9:.1f} GB", flush=True)
    wl = w.named(name, shape)
    pool_t = torch.empty((shape.n_planes, shape.n_pages, shape.tile_bytes), dtype=torch.uint8, device=cuda)
    _fill(pool_t)
    scale_t = None
    if shape.scales:
        scale_t = torch.empty((shape.n_planes, shape.n_pages, shape.scale_tile_bytes), dtype=torch.uint8, device=cuda)
        _fill(scale_t)
    pool = bk.PagedKVPool.from_stacked(pool_t, plane_dims=1, scale=scale_t)
    cap_pages = int(12e9 // shape.page_bytes)
    planes = sorted({0, 1, shape.n_planes // 2, shape.n_planes - 1})

    # gather (duplicates and out-of-order ids included, as the workload has them)
    g_reqs = _cap(wl["gather"], cap_pages)
    gb = pool.make_batch(g_reqs, layout)
    st, sc = pool.gather(gb)
    pool.check()
    _check_against_index_select(pool_t, st, gb, g_reqs, planes)
    if scale_t is not None:
        _check_against_index_select(scale_t, sc, gb, g_reqs, planes)
    allg = np.concatenate(g_reqs)
    uniq, first, counts = np.unique(allg, return_index=True, return_counts=True)
    if (counts > 1).any():          # a duplicated id gives identical rows wherever it appears
        pid = uniq[counts > 1][0]
        where = np.flatnonzero(allg == pid)[:2]
        rows = []
        owner = np.repeat(np.arange(len(g_reqs)), [len(r) for r in g_reqs])
        starts = np.concatenate([[0], np.cumsum([len(r) for r in g_reqs])])
        for i in where:
            r = owner[i]
            v = gb.request_view(st, int(r))
            j = int(i - starts[r])
            rows.append(v[:, j] if layout == "layer_major" else v[j])
        assert torch.equal(rows[0], rows[1])

    # scatter the gathered bytes into fresh pages, then read them back
    used = set(allg.tolist())
    fresh = np.array([p for p in np.random.default_rng(77).permutation(shape.n_pages) if p not in used][: len(allg)],
                     dtype=np.int64)
    if len(fresh) == len(allg):
        cuts = np.cumsum([len(r) for r in g_reqs])[:-1]
        s_reqs = [np.ascontiguousarray(a) for a in np.split(fresh, cuts)]
        untouched = np.setdiff1d(np.arange(shape.n_pages), fresh)[:4096]
        ut = torch.from_numpy(untouched).to(cuda)
        before = [pool_t[q, ut].to(torch.int64).sum().item() for q in planes]
        sb = pool.make_batch(s_reqs, layout)
        pool.scatter(sb, st, sc)
        pool.check()
        st2, sc2 = pool.gather(sb)
        pool.check()
        assert torch.equal(st2, st)
        if sc is not None:
            assert torch.equal(sc2, sc)
        _check_against_index_select(pool_t, st, sb, s_reqs, planes)
        after = [pool_t[q, ut].to(torch.int64).sum().item() for q in planes]
        assert before == after
    pool.close()
    del pool_t, scale_t, st, sc
    torch.cuda.empty_cache()
