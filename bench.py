#!/usr/bin/env python3
"""Benchmark of the KV page-copy hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload qwen2_7b|qwen2_1p5b|llama3_8b|
                    llama3_70b_fp8|reference_200x50]

Default workload = the configuration the headline target is quoted on: the Qwen2-7B-shaped bf16 pool
(28 layers x K/V, 131072 pages of 16 tokens x 4 heads x 128, ~120 GB resident in HBM) with 64
requests of 1024..8192 tokens, half gathered into contiguous per-request staging buffers, half
scattered from contiguous received buffers into freshly allocated pages, ~10 % of the gather ids
shared between requests. One step = one gather launch + one scatter launch over the whole batch.
Inputs (pool, staging, index arrays) are resident in HBM before the timed region starts.

Prints ONE JSON line. `value` = algorithmic bytes (payload read + payload written) per second over
the timed steps; `roofline` prices the slower of the two kernels against 8 TB/s with the launch
durations measured here with HIP events on the launch stream; `cpu_baseline` times the reference's
CPU path (torch.index_select / index_copy_ on host tensors) on this box's cores on a bounded sample
of the same request stream.

`llama3_8b` additionally runs the per-request gather -> pinned-host staging pipeline and reports
host-link GB/s next to a plain hipMemcpyAsync of one large pinned buffer measured in the same run.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [ROOT, os.path.join(ROOT, "bi-kv_amd")]

HBM_PEAK_GBPS = 8000.0

# HBM bytes per launch as a multiple of the algorithmic bytes, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of this file, each scaled by the same counter's reading for the plain-copy
# calibration launch below (summaries under profiles/). None = not measured for that workload.
MEASURED_TRAFFIC_RATIO = {"qwen2_7b": {"gather": 0.9949, "scatter": 1.0003},
                          "qwen2_7b_token_major": {"gather": 0.9997, "scatter": 1.0002},
                          "layout_change": {"load": 1.0035, "store": 1.0029}}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="qwen2_7b")
    ap.add_argument("--layout", default="layer_major", choices=["layer_major", "page_major"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-layout", dest="no_other_layout", action="store_true",
                    help="skip the second measurement with the other staging layout")
    ap.add_argument("--pool-pages", type=int, default=0, help="override the pool size (pages per plane)")
    ap.add_argument("--pool-alloc", choices=["planes", "stacked"], default="stacked",
                    help="one device tensor per (layer, K|V) plane, or one stacked allocation")
    ap.add_argument("--seg", type=int, default=None)
    ap.add_argument("--unroll", type=int, default=None)
    ap.add_argument("--nontemporal", type=int, default=None)
    ap.add_argument("--wave-block", dest="wave_block", type=int, default=None)
    ap.add_argument("--order", type=int, default=None)
    ap.add_argument("--log2-chunk", dest="log2_chunk", type=int, default=None)
    ap.add_argument("--staging-cap-gb", dest="staging_cap_gb", type=float, default=32.0,
                    help="largest staging buffer of one launch; bigger batches take several launches")
    ap.add_argument("--chunk-mib", type=int, default=32, help="staging pipeline chunk (llama3_8b)")
    ap.add_argument("--buffers", type=int, default=2, help="staging pipeline lanes (stream + HBM chunk each)")
    return ap.parse_args()


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def fill_random_bytes(t):
    """Random bytes in place, one plane at a time (bit patterns are what matters for a byte mover)."""
    import torch
    flat = t.view(torch.uint8).reshape(-1)
    step = 1 << 31
    for off in range(0, flat.numel(), step):
        flat[off: off + step].random_(0, 256)


def make_pool(shape, dev, alloc="planes"):
    """The pool as the serving engine holds it: one tensor per (layer, K|V) plane ("planes", as
    Bi-KV/Worker/Worker.py:74-78 keeps a list of per-layer caches), or one stacked allocation
    ("stacked"). Returns (planes, scale planes or None); both index as planes[q] -> [n_pages, tile]."""
    import torch

    def one(tile_bytes):
        if alloc == "stacked":
            t = torch.empty((shape.n_planes, shape.n_pages, tile_bytes), dtype=torch.uint8, device=dev)
            fill_random_bytes(t)
            return [t[q] for q in range(shape.n_planes)]
        out = [torch.empty((shape.n_pages, tile_bytes), dtype=torch.uint8, device=dev) for _ in range(shape.n_planes)]
        for t in out:
            fill_random_bytes(t)
        return out

    return one(shape.tile_bytes), (one(shape.scale_tile_bytes) if shape.scales else None)


def verify_on_device(pool_t, staging, batch, requests, n_check_planes=3):
    """Independent check at full size: torch.index_select on the device, a few planes per request."""
    import torch
    n_planes = len(pool_t)
    planes = sorted({0, n_planes // 2, n_planes - 1})[:n_check_planes]
    for r, ids in enumerate(requests):
        if len(ids) == 0:
            continue
        view = batch.request_view(staging, r)
        idt = torch.from_numpy(ids).to(pool_t[0].device)
        for q in planes:
            want = torch.index_select(pool_t[q], 0, idt)
            got = view[q] if batch.layout == "layer_major" else view[:, q]
            if not torch.equal(got, want):
                return False
    return True


def time_plain_copy(bk, dev, nbytes=2 << 30, iters=5):
    """A plain contiguous copy through the run-copy kernel: the achievable-bandwidth yardstick and the
    known-size launch that calibrates the FETCH_SIZE / WRITE_SIZE counters."""
    import torch
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    src.random_(0, 256)
    dst = torch.empty_like(src)
    zero = torch.zeros(1, dtype=torch.int64, device=dev)
    bk.copy_runs(src, dst, zero, zero, nbytes)
    torch.cuda.synchronize(dev)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        bk.copy_runs(src, dst, zero, zero, nbytes)
    e1.record()
    torch.cuda.synchronize(dev)
    ms = e0.elapsed_time(e1) / iters
    ok = torch.equal(src, dst)
    del src, dst
    return 2 * nbytes / (ms * 1e-3) / 1e9, ok


def cpu_baseline(shape, wl, budget_s=12.0):
    """The reference's CPU path on this box's cores: torch.index_select (gather) and index_copy_
    (scatter) on host tensors [planes, pages, tile]. The host pool is capped (page ids are reduced
    modulo its page count) and only the leading requests are replayed; passes are repeated for about
    `budget_s` seconds of CPU work and the median pass is reported."""
    import numpy as np
    import torch
    from oracle import pagecopy_oracle as oracle

    threads = torch.get_num_threads()
    host_bytes_cap = 8 << 30
    try:
        import psutil
        host_bytes_cap = min(host_bytes_cap, int(psutil.virtual_memory().total * 0.25))
    except Exception:
        pass
    host_pages = max(64, min(shape.n_pages, host_bytes_cap // (shape.tile_bytes * shape.n_planes)))
    pool = torch.empty((shape.n_planes, host_pages, shape.tile_bytes), dtype=torch.uint8)
    pool.view(torch.int64).reshape(-1).copy_(torch.arange(pool.numel() // 8, dtype=torch.int64))
    g_reqs = [torch.from_numpy(np.ascontiguousarray(r % host_pages)) for r in wl["gather"]]
    s_src = wl.get("scatter") or wl["gather"]
    # unique destinations inside the capped pool: take distinct ids from a permutation
    perm = np.random.default_rng(1234).permutation(host_pages)
    page_cap = 4096                                   # pages per direction in the sample
    g_sel, used = [], 0
    for r in g_reqs:
        if used + len(r) > page_cap and g_sel:
            break
        g_sel.append(r)
        used += len(r)
    s_sel, s_used = [], 0
    for r in s_src:
        n = min(len(r), host_pages - s_used)
        if n <= 0 or (s_used + n > page_cap and s_sel):
            break
        s_sel.append(torch.from_numpy(np.ascontiguousarray(perm[s_used: s_used + n])))
        s_used += n
    outs = [torch.empty((shape.n_planes, len(r), shape.tile_bytes), dtype=torch.uint8) for r in g_sel]
    srcs = [torch.empty((shape.n_planes, len(r), shape.tile_bytes), dtype=torch.uint8).fill_(3) for r in s_sel]

    def one_pass():
        for ids, out in zip(g_sel, outs):
            oracle.gather_layered_torch(pool, ids, out)
        for ids, src in zip(s_sel, srcs):
            oracle.scatter_layered_torch(pool, ids, src)

    one_pass()                                        # warm-up (also faults the pages in)
    times = []
    t_start = time.perf_counter()
    while len(times) < 5 or ((time.perf_counter() - t_start) < budget_s and len(times) < 60):
        t0 = time.perf_counter()
        one_pass()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    pages = used + s_used
    alg_bytes = 2 * pages * shape.tile_bytes * shape.n_planes
    return {
        "value": round(alg_bytes / med / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": (f"torch.index_select + index_copy_ on host tensors, {len(g_sel)} gather + {len(s_sel)} "
                   f"scatter requests ({pages} pages, {alg_bytes / 1e9:.2f} GB read+written per pass), host pool "
                   f"capped to {host_pages} pages/plane with ids modulo that, median of {len(times)} passes "
                   f"({sum(times):.1f} s of CPU work)"),
        "pages_per_s": round(pages / med, 1),
    }


def run_gather_scatter(args, bk, workloads, dev, with_copy=True):
    import numpy as np
    import torch

    name = args.workload
    shape = workloads.SHAPES[name]
    if args.pool_pages:
        shape = shape.scaled(args.pool_pages)
    wl = workloads.named(name, shape)
    log(f"{name}: pool {shape.pool_bytes / 1e9:.2f} GB, tile {shape.tile_bytes} B x {shape.n_planes} planes")
    pool_t, scale_t = make_pool(shape, dev, args.pool_alloc)
    pool = bk.PagedKVPool.from_planes(pool_t, scale_t)

    g_reqs = wl["gather"]
    s_reqs = wl.get("scatter") or []

    # A launch covers as many whole requests as fit a staging buffer of --staging-cap-gb; the
    # Qwen2-7B-shaped batch fits in one launch per direction, the 70B-shaped one needs a few.
    def groups_of(reqs):
        cap_pages = max(1, int(args.staging_cap_gb * 1e9) // shape.page_bytes)
        out, cur, used = [], [], 0
        for r in reqs:
            if cur and used + len(r) > cap_pages:
                out.append(cur)
                cur, used = [], 0
            cur.append(r)
            used += len(r)
        if cur:
            out.append(cur)
        return [(pool.make_batch(g, args.layout), g) for g in out]

    g_groups, s_groups = groups_of(g_reqs), groups_of(s_reqs)
    max_slots = max(b.n_slots for b, _ in g_groups + s_groups)
    g_st = torch.empty(max_slots * shape.tile_bytes, dtype=torch.uint8, device=dev)
    g_sc = torch.empty(max_slots * shape.scale_tile_bytes, dtype=torch.uint8, device=dev) if shape.scales else None
    s_st = s_sc = None
    if s_groups:
        s_st = torch.empty_like(g_st)
        fill_random_bytes(s_st)
        if shape.scales:
            s_sc = torch.empty_like(g_sc)
            fill_random_bytes(s_sc)

    def views(batch, st, sc):
        return (st[: batch.n_slots * shape.tile_bytes],
                sc[: batch.n_slots * shape.scale_tile_bytes] if sc is not None else None)

    torch.cuda.synchronize(dev)
    g_pages = sum(b.n_pages for b, _ in g_groups)
    s_pages = sum(b.n_pages for b, _ in s_groups)
    n_pages = g_pages + s_pages
    alg_g = 2 * g_pages * shape.page_bytes
    alg_s = 2 * s_pages * shape.page_bytes
    log(f"gather {g_pages} pages in {len(g_groups)} launch(es) ({alg_g / 1e9:.2f} GB r+w), scatter {s_pages} pages in "
        f"{len(s_groups)} launch(es) ({alg_s / 1e9:.2f} GB r+w)")

    def step(events=None):
        if events is not None:
            events[0].record()
        for b, _ in g_groups:
            pool.gather(b, *views(b, g_st, g_sc))
        if events is not None:
            events[1].record()
        for b, _ in s_groups:
            pool.scatter(b, *views(b, s_st, s_sc))
        if events is not None:
            events[2].record()

    for _ in range(args.warmup):
        step()
    pool.check()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for k in range(args.steps):
        step(evs[k])
    torch.cuda.synchronize(dev)
    wall = time.perf_counter() - t0
    pool.check()

    # per-launch averages (a direction's launches are back to back between two events)
    g_ms = [e[0].elapsed_time(e[1]) / len(g_groups) for e in evs]
    s_ms = [e[1].elapsed_time(e[2]) / max(1, len(s_groups)) for e in evs]
    ms_per_step = wall * 1e3 / args.steps
    value = (alg_g + alg_s) / (wall / args.steps) / 1e9
    g_gbps = alg_g / len(g_groups) / (np.mean(g_ms) * 1e-3) / 1e9
    s_gbps = alg_s / len(s_groups) / (np.mean(s_ms) * 1e-3) / 1e9 if s_groups else None
    sb = s_groups or None

    # parity at full size, outside the timed region: scattered pages must equal their source, and
    # each gather launch is repeated and checked against torch.index_select on the device
    ok = True
    for b, reqs in s_groups:
        st, sc = views(b, s_st, s_sc)
        ok = ok and verify_on_device(pool_t, st, b, reqs)
        if scale_t is not None:
            ok = ok and verify_on_device(scale_t, sc, b, reqs)
    for b, reqs in g_groups:
        st, sc = views(b, g_st, g_sc)
        st.zero_()
        pool.gather(b, st, sc)
        pool.check()
        ok = ok and verify_on_device(pool_t, st, b, reqs)
        if scale_t is not None:
            ok = ok and verify_on_device(scale_t, sc, b, reqs)
    if not ok:
        raise SystemExit("bench: results differ from torch.index_select on the device — not reporting")
    alg_g //= len(g_groups)          # per launch, for the roofline entries below
    alg_s //= max(1, len(s_groups))

    copy_gbps, copy_ok = time_plain_copy(bk, dev) if with_copy else (0.0, True)
    if not copy_ok:
        raise SystemExit("bench: plain copy mismatch")

    # the dominant kernel = the instantiation that takes more of the step
    dominant_is_gather = (s_gbps is None) or (float(np.sum(g_ms)) >= float(np.sum(s_ms)))
    kname = "bikv::tile_move_wave_kernel<0=gather>" if dominant_is_gather else "bikv::tile_move_wave_kernel<1=scatter>"
    ach = g_gbps if dominant_is_gather else s_gbps
    alg_dom = alg_g if dominant_is_gather else alg_s
    ms_dom = float(np.mean(g_ms if dominant_is_gather else s_ms))
    ratio = MEASURED_TRAFFIC_RATIO.get(name, {}).get("gather" if dominant_is_gather else "scatter")
    if args.pool_pages or args.layout != "layer_major":
        ratio = None                                   # measured on the full-size default workload only
    out = {
        "metric": "paged-KV gather/scatter HBM GB/s (% of MI355X peak) + pages/s, bit-exact",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": f"{name}: {shape.layers} layers x K/V, {shape.n_pages} pages x {shape.page_tokens} tok x "
                               f"{shape.kv_heads} heads x {shape.head_dim} {shape.dtype}"
                               f"{' + fp32 scales' if shape.scales else ''}; {len(g_reqs)} gather + {len(s_reqs)} "
                               f"scatter requests, {n_pages} pages/step in {len(g_groups)}+{len(s_groups)} launches, "
                               f"layout {args.layout}",
                   "pool_GB": round(shape.pool_bytes / 1e9, 2), "tile_bytes": shape.tile_bytes,
                   "planes": shape.n_planes, "pool_alloc": args.pool_alloc},
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "pages_per_s": round(n_pages / (wall / args.steps), 1),
        "bit_exact": True,
        "roofline": {"bound": "hbm", "kernel": kname, "achieved": round(ach, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBPS, 4),
                     "traffic": (round(ratio * alg_dom) if ratio else None),
                     "alg_bytes_per_launch": alg_dom, "avg_launch_ms": round(ms_dom, 4)},
        "kernels": {"gather": {"GBps": round(g_gbps, 1), "avg_ms": round(float(np.mean(g_ms)), 4),
                               "min_ms": round(float(np.min(g_ms)), 4), "alg_bytes": alg_g},
                    "scatter": ({"GBps": round(s_gbps, 1), "avg_ms": round(float(np.mean(s_ms)), 4),
                                 "min_ms": round(float(np.min(s_ms)), 4), "alg_bytes": alg_s} if sb else None),
                    "plain_copy_2GiB": ({"GBps": round(copy_gbps, 1)} if with_copy else None)},
    }
    del pool_t, scale_t, g_st, s_st
    torch.cuda.empty_cache()
    return out, shape, wl


def run_staging(args, bk, workloads, dev):
    """llama3_8b: per-request gather followed by the device -> pinned-host copy, overlapped in chunks."""
    import numpy as np
    import torch

    shape = workloads.SHAPES["llama3_8b"]
    if args.pool_pages:
        shape = shape.scaled(args.pool_pages)
    wl = workloads.named("llama3_8b", shape)
    pool_t, _ = make_pool(shape, dev, args.pool_alloc)
    pool = bk.PagedKVPool.from_planes(pool_t)
    reqs = wl["gather"]
    max_pages = max(len(r) for r in reqs)
    host = bk.pinned_empty(max_pages * shape.page_bytes)
    host.zero_()
    # host-link yardstick: one large pinned buffer, plain hipMemcpyAsync
    dev_buf = torch.empty(min(host.numel(), 1 << 30), dtype=torch.uint8, device=dev)
    dev_buf.random_(0, 256)
    # the first DMA into a pinned page is slower than later ones: touch the whole buffer once
    for off in range(0, host.numel(), dev_buf.numel()):
        n = min(dev_buf.numel(), host.numel() - off)
        host[off: off + n].copy_(dev_buf[:n])
    link = []
    for _ in range(4):
        link.append(dev_buf.numel() / bk.measure_d2h(dev, host, dev_buf, 0) / 1e9)
    link_gbps = max(link[1:])
    up = []
    for _ in range(4):
        up.append(dev_buf.numel() / bk.measure_h2d(dev, dev_buf, host, 0) / 1e9)
    up_gbps = max(up[1:])
    results = {}
    for mode in ("pipelined", "direct"):
        stager = bk.HostStager(dev, chunk_bytes=args.chunk_mib << 20, n_buffers=args.buffers)
        batches = [pool.make_batch([r], args.layout) for r in reqs]
        torch.cuda.synchronize(dev)
        stager.gather_to_host(pool, batches[0], host, mode)      # warm-up
        tot_b, tot_s, chunks = 0, 0.0, 0
        for b in batches[: max(1, args.steps)]:
            nb, nc, sec = stager.gather_to_host(pool, b, host, mode)
            tot_b += nb
            tot_s += sec
            chunks += nc
        # parity of the last request staged
        b = batches[max(1, args.steps) - 1 if args.steps <= len(batches) else -1]
        stager.gather_to_host(pool, b, host, mode)
        r = reqs[batches.index(b)]
        idt = torch.from_numpy(r).to(dev)
        view = host[: b.n_slots * shape.tile_bytes].view(b.n_slots, shape.tile_bytes)
        ok = True
        for q in (0, shape.n_planes - 1):
            want = torch.index_select(pool_t[q], 0, idt).cpu()
            got = view[q * len(r): (q + 1) * len(r)] if args.layout == "layer_major" else view[q::shape.n_planes]
            ok = ok and torch.equal(got, want)
        if not ok:
            raise SystemExit(f"bench: staged bytes differ ({mode})")
        results[mode] = {"host_link_GBps": round(tot_b / tot_s / 1e9, 2), "bytes": tot_b, "chunks": chunks,
                         "frac_of_plain_d2h": round(tot_b / tot_s / 1e9 / link_gbps, 4)}
        # the receiving side: the staged image of a request goes host -> pool, into the pages next to
        # the ones it came from (a different, still unique id set)
        rx_b, rx_s = 0, 0.0
        rx = [(b_, r_) for b_, r_ in zip(batches, reqs) if len(np.unique(r_)) == len(r_)][: max(1, args.steps)]
        for b_, r_ in rx:
            stager.gather_to_host(pool, b_, host, mode)
            shifted = (np.asarray(r_) + 1) % shape.n_pages
            sb = pool.make_batch([shifted], args.layout)
            nb, _, sec = stager.scatter_from_host(pool, sb, host, mode)
            rx_b += nb
            rx_s += sec
        if rx:
            idt = torch.from_numpy(shifted).to(dev)
            view = host[: sb.n_slots * shape.tile_bytes].view(sb.n_slots, shape.tile_bytes)
            for q in (0, shape.n_planes - 1):
                got = torch.index_select(pool_t[q], 0, idt).cpu()
                want = (view[q * len(shifted): (q + 1) * len(shifted)] if args.layout == "layer_major"
                        else view[q::shape.n_planes])
                if not torch.equal(got, want):
                    raise SystemExit(f"bench: scattered bytes differ ({mode})")
            results[mode]["scatter_from_host_GBps"] = round(rx_b / rx_s / 1e9, 2)
            results[mode]["scatter_frac_of_plain_h2d"] = round(rx_b / rx_s / 1e9 / up_gbps, 4)
        stager.close()
    return {"plain_d2h_GBps": round(link_gbps, 2), "plain_h2d_GBps": round(up_gbps, 2),
            "chunk_MiB": args.chunk_mib, "buffers": args.buffers,
            "requests": min(len(reqs), max(1, args.steps)), **results}


def run_reference_scenario(args, bk, dev):
    """The only workload the reference itself scripts: 200 pages x 50 tokens x 14336 fp16 elements,
    identity offsets, one run copy per transfer (test_page_ipc.py:41-65)."""
    import torch
    page_elements = 50 * 128 * 2 * 28 * 2
    n = 200
    cache = torch.full((n * page_elements,), 7, dtype=torch.float16, device=dev)
    out = torch.empty_like(cache)
    offs = torch.arange(n, dtype=torch.int64, device=dev) * page_elements
    for _ in range(args.warmup):
        bk.copy_runs(cache, out, offs, offs, page_elements)
    torch.cuda.synchronize(dev)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        bk.copy_runs(cache, out, offs, offs, page_elements)
    e1.record()
    torch.cuda.synchronize(dev)
    wall = time.perf_counter() - t0
    if not torch.equal(out, cache):
        raise SystemExit("bench: reference scenario mismatch")
    alg = 2 * cache.numel() * 2
    ms = e0.elapsed_time(e1) / args.steps
    # the zero-copy form of the same scenario (test_zero_copy.py:40-56): the pool is pinned host memory
    # and the kernel reads it over the host link; yardstick = a plain pinned H2D copy of the same bytes
    pinned = torch.full((n * page_elements,), 7, dtype=torch.float16).pin_memory()
    out.zero_()
    bk.copy_runs(pinned, out, offs, offs, page_elements, device=dev)
    out.copy_(pinned, non_blocking=True)
    torch.cuda.synchronize(dev)
    zc, h2d = [], []
    for _ in range(max(3, args.steps // 4)):
        e0.record()
        bk.copy_runs(pinned, out, offs, offs, page_elements, device=dev)
        e1.record()
        torch.cuda.synchronize(dev)
        zc.append(e0.elapsed_time(e1))
        e0.record()
        out.copy_(pinned, non_blocking=True)
        e1.record()
        torch.cuda.synchronize(dev)
        h2d.append(e0.elapsed_time(e1))
    if not torch.equal(out, cache):
        raise SystemExit("bench: zero-copy scenario mismatch")
    nbytes = cache.numel() * 2
    zero_copy = {"GBps": round(nbytes / (min(zc) * 1e-3) / 1e9, 2),
                 "plain_pinned_h2d_GBps": round(nbytes / (min(h2d) * 1e-3) / 1e9, 2)}
    # the same launches captured once in a HIP graph and replayed: what a serving loop pays per transfer
    # once the Python and launch overhead is taken out of the loop
    out.zero_()
    side = torch.cuda.Stream(device=dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for _ in range(args.steps):
                bk.copy_runs(cache, out, offs, offs, page_elements)
    graph.replay()
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    graph.replay()
    torch.cuda.synchronize(dev)
    graph_wall = time.perf_counter() - t0
    if not torch.equal(out, cache):
        raise SystemExit("bench: graph replay mismatch")
    return {
        "zero_copy_from_pinned_host": zero_copy,
        "graph_replay": {"GBps": round(alg / (graph_wall / args.steps) / 1e9, 1),
                         "ms_per_launch": round(graph_wall * 1e3 / args.steps, 4)},
        "metric": "paged-KV gather/scatter HBM GB/s (% of MI355X peak) + pages/s, bit-exact",
        "value": round(alg / (wall / args.steps) / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall * 1e3 / args.steps, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": "reference_200x50: 200 pages x 50 tokens x 14336 fp16, identity offsets, value 7"},
        "pages_per_s": round(n / (wall / args.steps), 1), "bit_exact": True,
        "roofline": {"bound": "hbm", "kernel": "bikv::copy_runs_wave_kernel", "achieved": round(alg / (ms * 1e-3) / 1e9, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                     "traffic": None, "alg_bytes_per_launch": alg, "avg_launch_ms": round(ms, 4)},
    }


def run_token_major(args, bk, workloads, dev):
    """The Qwen2-7B request stream in the REFERENCE'S layout: a token-major pool of 131072 pages of
    16 tokens x (128, 4, 28, 2) bf16 = 917 504 bytes each (kvcache.py:38-43 at this shape), one run per
    page through the run copy (block_per_page_copy_kernel's role, copy_kernel.cu:9-36): gather the 32
    gather requests into a dense buffer, scatter the 32 scatter requests back from it."""
    import numpy as np
    import torch
    shape = workloads.SHAPES["qwen2_7b"]
    if args.pool_pages:
        shape = shape.scaled(args.pool_pages)
    wl = workloads.named("qwen2_7b", shape)
    page_elems = shape.page_bytes // 2
    pool = torch.empty(shape.n_pages * page_elems, dtype=torch.bfloat16, device=dev)
    fill_random_bytes(pool)
    g_ids = np.concatenate(wl["gather"]).astype(np.int64)
    s_ids = np.concatenate(wl["scatter"]).astype(np.int64)
    n_g, n_s = len(g_ids), len(s_ids)
    dense = torch.empty(max(n_g, n_s) * page_elems, dtype=torch.bfloat16, device=dev)
    g_src = torch.from_numpy(g_ids * page_elems).to(dev)
    s_dst = torch.from_numpy(s_ids * page_elems).to(dev)
    g_dst = torch.arange(n_g, dtype=torch.int64, device=dev) * page_elems
    s_src = torch.arange(n_s, dtype=torch.int64, device=dev) * page_elems

    def step(ev=None):
        if ev:
            ev[0].record()
        bk.copy_runs(pool, dense, g_src, g_dst, page_elems)
        if ev:
            ev[1].record()
        bk.copy_runs(dense, pool, s_src, s_dst, page_elems)
        if ev:
            ev[2].record()

    # parity of the gather at full size: torch.index_select over the page view
    bk.copy_runs(pool, dense, g_src, g_dst, page_elems)
    from bikv_pagecopy import runs
    runs.check(dev)
    view = pool.view(torch.int16).view(shape.n_pages, page_elems)
    sample = np.arange(0, n_g, max(1, n_g // 64))
    want = torch.index_select(view, 0, torch.from_numpy(g_ids[sample]).to(dev))
    got = dense.view(torch.int16).view(-1, page_elems)[torch.from_numpy(sample).to(dev)]
    if not torch.equal(got, want):
        raise SystemExit("bench: token-major gather differs from torch.index_select")
    for _ in range(args.warmup):
        step()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for k in range(args.steps):
        step(evs[k])
    torch.cuda.synchronize(dev)
    wall = time.perf_counter() - t0
    runs.check(dev)
    # the scatter wrote the dense buffer's first n_s pages into the scatter ids
    got = torch.index_select(view, 0, torch.from_numpy(s_ids[:64]).to(dev))
    if not torch.equal(got, dense.view(torch.int16).view(-1, page_elems)[:64]):
        raise SystemExit("bench: token-major scatter differs")
    g_ms = float(np.mean([e[0].elapsed_time(e[1]) for e in evs]))
    s_ms = float(np.mean([e[1].elapsed_time(e[2]) for e in evs]))
    alg_g, alg_s = 2 * n_g * shape.page_bytes, 2 * n_s * shape.page_bytes
    slow_g = alg_g / g_ms <= alg_s / s_ms
    alg, ms = (alg_g, g_ms) if slow_g else (alg_s, s_ms)
    value = (alg_g + alg_s) / (wall / args.steps) / 1e9
    return {
        "metric": "paged-KV gather/scatter HBM GB/s (% of MI355X peak) + pages/s, bit-exact",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3 / args.steps, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": f"qwen2_7b_token_major: {shape.n_pages} pages x {shape.page_bytes} B (16 tok x (128,4,28,2) bf16), "
                               f"{n_g} pages gathered + {n_s} scattered per step, one run per page",
                   "pool_GB": round(shape.pool_bytes / 1e9, 2)},
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "pages_per_s": round((n_g + n_s) / (wall / args.steps), 1), "bit_exact": True,
        "kernels": {"gather": {"GBps": round(alg_g / g_ms / 1e6, 1), "avg_ms": round(g_ms, 4)},
                    "scatter": {"GBps": round(alg_s / s_ms / 1e6, 1), "avg_ms": round(s_ms, 4)}},
        "roofline": {"bound": "hbm", "kernel": "bikv::copy_runs_wave_kernel", "achieved": round(alg / ms / 1e6, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(alg / ms / 1e6 / HBM_PEAK_GBPS, 4),
                     "traffic": (int(alg * MEASURED_TRAFFIC_RATIO["qwen2_7b_token_major"]["gather" if slow_g else "scatter"])
                                 if not args.pool_pages else None),
                     "alg_bytes_per_launch": alg, "avg_launch_ms": round(ms, 4)},
    }


def run_layout_change(args, bk, dev):
    """Received token-major pages -> the Worker's per-layer paged pool and back, at the reference's own
    shapes: token_shape (128, 2, 28, 2) fp16 (Model/qwen2.py:512-522), 28 layer tensors of
    [10240*16, 2, 2, 128] (Worker.py:69-78), 4096 pages of 16 tokens per step and direction."""
    import numpy as np
    import torch
    from oracle import pagecopy_oracle as oracle

    P, D, H, L, blocks, n_pages = 16, 128, 2, 28, 10240, 4096
    if args.pool_pages:
        blocks = args.pool_pages
        n_pages = min(n_pages, blocks)
    layers = [torch.empty((blocks * P, 2, H, D), dtype=torch.float16, device=dev) for _ in range(L)]
    for t in layers:
        fill_random_bytes(t)
    pool = bk.NHDPool.from_token_kv_layers(layers, P)
    tm = torch.empty((n_pages, P, D, H, L, 2), dtype=torch.float16, device=dev)
    fill_random_bytes(tm)
    tm_out = torch.empty_like(tm)
    rng = np.random.default_rng(6)
    ids_h = rng.permutation(blocks)[:n_pages].astype(np.int64)
    ids = torch.from_numpy(ids_h).to(dev)
    alg = 2 * tm.numel() * 2                       # bytes read + written per launch

    def step(ev=None):
        if ev:
            ev[0].record()
        pool.load_token_major(tm, ids)             # received pages -> pool blocks
        if ev:
            ev[1].record()
        pool.store_token_major(tm_out, ids)        # the same blocks -> pages to send
        if ev:
            ev[2].record()

    for _ in range(args.warmup):
        step()
    pool.check()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for k in range(args.steps):
        step(evs[k])
    torch.cuda.synchronize(dev)
    wall = time.perf_counter() - t0
    pool.check()
    if not torch.equal(tm_out.view(torch.int16), tm.view(torch.int16)):
        raise SystemExit("bench: store(load(x)) != x")
    # a sample of pages against the CPU oracle
    sample = np.arange(0, n_pages, max(1, n_pages // 8))[:8]
    lay_h = [np.zeros((blocks * P, 2, H, D), dtype=np.uint16) for _ in range(L)]
    tm_h = tm[torch.from_numpy(sample).to(dev)].cpu().view(torch.int16).numpy().view(np.uint16)
    oracle.transpose_pages_c(lay_h, "token_kv", np.ascontiguousarray(tm_h), ids_h[sample], np.arange(len(sample)), "load")
    for l in (0, L // 2, L - 1):
        for b in ids_h[sample]:
            got = layers[l][b * P:(b + 1) * P].cpu().view(torch.int16).numpy().view(np.uint16)
            if got.tobytes() != lay_h[l][b * P:(b + 1) * P].tobytes():
                raise SystemExit("bench: layout change differs from the oracle")
    l_ms = [e[0].elapsed_time(e[1]) for e in evs]
    s_ms = [e[1].elapsed_time(e[2]) for e in evs]
    slow_is_load = np.mean(l_ms) >= np.mean(s_ms)
    ms_dom = float(np.mean(l_ms if slow_is_load else s_ms))
    return {
        "metric": "paged-KV gather/scatter HBM GB/s (% of MI355X peak) + pages/s, bit-exact",
        "value": round(2 * alg / (wall / args.steps) / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall * 1e3 / args.steps, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u16", "data": "synthetic",
        "config": {"workload": f"layout_change: token-major pages <-> {L} layer tensors [{blocks}*{P}, 2, {H}, {D}] fp16, "
                               f"{n_pages} pages of {P} tokens loaded then stored per step"},
        "pct_of_hbm_peak": round(100 * 2 * alg / (wall / args.steps) / 1e9 / HBM_PEAK_GBPS, 2),
        "pages_per_s": round(2 * n_pages / (wall / args.steps), 1), "bit_exact": True,
        "roofline": {"bound": "hbm", "kernel": f"bikv::transpose_pairs_kernel<{1 if slow_is_load else 0}, 2, 512>",
                     "achieved": round(alg / (ms_dom * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(alg / (ms_dom * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                     "traffic": (int(alg * MEASURED_TRAFFIC_RATIO["layout_change"]["load" if slow_is_load else "store"])
                                 if not args.pool_pages else None),
                     "alg_bytes_per_launch": alg, "avg_launch_ms": round(ms_dom, 4)},
        "kernels": {"load": {"GBps": round(alg / (np.mean(l_ms) * 1e-3) / 1e9, 1), "avg_ms": round(float(np.mean(l_ms)), 4)},
                    "store": {"GBps": round(alg / (np.mean(s_ms) * 1e-3) / 1e9, 1), "avg_ms": round(float(np.mean(s_ms)), 4)}},
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no cross-GPU step (pages are independent; each GPU "
              "gathers/scatters its own pool). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch
    import __graft_entry__ as entry
    entry.ensure_built()
    import bikv_pagecopy as bk
    from bikv_pagecopy import workloads

    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU: the page-copy path has no CPU fallback")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    knobs = {k: getattr(args, k) for k in ("seg", "unroll", "nontemporal", "wave_block", "order", "log2_chunk") if getattr(args, k) is not None}
    if knobs:
        bk.set_tuning(**knobs)

    if args.workload == "reference_200x50":
        out = run_reference_scenario(args, bk, dev)
        print(json.dumps(out), flush=True)
        return
    if args.workload == "qwen2_7b_token_major":
        out = run_token_major(args, bk, workloads, dev)
        print(json.dumps(out), flush=True)
        return
    if args.workload == "layout_change":
        out = run_layout_change(args, bk, dev)
        print(json.dumps(out), flush=True)
        return
    out, shape, wl = run_gather_scatter(args, bk, workloads, dev)
    if knobs:
        out["config"]["tuning"] = knobs
    if not args.no_other_layout:
        # the same request stream with the other staging image (reported next to the headline number)
        import copy
        alt = copy.copy(args)
        alt.layout = "page_major" if args.layout == "layer_major" else "layer_major"
        alt.steps, alt.warmup = max(3, args.steps // 2), 2
        log(f"same workload, staging layout {alt.layout}")
        o2, _, _ = run_gather_scatter(alt, bk, workloads, dev, with_copy=False)
        out["other_layout"] = {"layout": alt.layout, "value": o2["value"], "pct_of_hbm_peak": o2["pct_of_hbm_peak"],
                               "steps": alt.steps, "kernels": {k: v for k, v in o2["kernels"].items() if v}}
    if args.workload == "llama3_8b":
        out["staging"] = run_staging(args, bk, workloads, dev)
    if not args.no_cpu_baseline:
        log("timing the CPU baseline")
        out["cpu_baseline"] = cpu_baseline(shape, wl)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
