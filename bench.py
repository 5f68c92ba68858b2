#!/usr/bin/env python3
"""Benchmark of the KV page-copy hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload qwen2_7b|qwen2_1p5b|llama3_8b|
                    llama3_70b_fp8|qwen2_7b_token_major|layout_change|staging|staging_trace|reference_200x50]
                    [--pool-form planar|worker] [--pool-alloc spread|stacked|planes] [--layout layer_major|page_major]

Default workload = the configuration the headline target is quoted on: the Qwen2-7B-shaped bf16 pool
(28 layers x K/V, 131072 pages of 16 tokens x 4 heads x 128, ~120 GB resident in HBM) with 64
requests of 1024..8192 tokens, half gathered into contiguous per-request staging buffers, half
scattered from contiguous received buffers into freshly allocated pages, ~10 % of the gather ids
shared between requests. One step = one gather launch + one scatter launch over the whole batch.
Inputs (pool, staging, index arrays) are resident in HBM before the timed region starts.

Prints ONE JSON line. `value` = algorithmic bytes (payload read + payload written) per second over
the timed steps (400 by default: about two seconds of back-to-back launches); `roofline` prices the
slower of the two kernels against 8 TB/s with the launch durations measured here with HIP events on
the launch stream (min / median / p99 per launch are in `kernels`); `cpu_baseline` times the
reference's CPU path (torch.index_select / index_copy_ on host tensors) on this box's cores on a
bounded sample of the same request stream.

The default run then measures, one after another at full pool size, the other named configurations
(`configs`: Qwen2-1.5B, Llama-3-8B, Llama-3-70B fp8 + scales) and, on the Llama-3-8B pool, the
pool <-> pinned-host staging pipeline (`staging`): all 128 requests enqueued back to back, 4-32 MiB
chunks on 2 lanes (3 and 4 lanes as contrast cases), kernel-direct and automatic modes, both directions, each next to a plain
hipMemcpyAsync of one large pinned buffer timed immediately before it. `--no-configs` / `--no-staging`
skip those parts.

`roofline.traffic` (HBM bytes per launch of the dominant kernel) is measured at the end of the default run: the
headline workload is run twice more as a child process under `rocprofv3 --pmc` (FETCH_SIZE, then WRITE_SIZE),
each counter scaled by its reading for the plain 2 GiB copy of the same child (`roofline.traffic_live`). If the
profiler is missing or a child fails, and with `--no-live-traffic`, the figure is the run's algorithmic bytes
times the ratio recorded from the same two commands under profiles/ (`traffic_source` says which).

Pools and gather destinations are allocated through the library's bikv_device_alloc, which lays their
physical chunks alternately in the two halves of HBM (`--pool-alloc torch` / `--staging-alloc torch`
take torch's allocator instead; the default run times the headline workload once more that way and
reports it as `torch_alloc`). If the library's allocator cannot serve a request the run falls back to
torch for that buffer and says so in `device_alloc`.
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
MEASURED_TRAFFIC_RATIO = {"qwen2_7b": {"gather": 0.9948, "scatter": 1.0002},
                          "qwen2_1p5b": {"gather": 1.0009},
                          "llama3_8b": {"gather": 0.9967},
                          "llama3_70b_fp8": {"gather": 1.0142, "scatter": 1.0002},
                          "qwen2_7b_token_major": {"gather": 0.9998, "scatter": 1.0002},
                          "layout_change": {"load": 1.0003, "store": 1.0022}}


# The ratios above describe the kernels as they were when the counters were read: the SHA-256 (first 16 hex
# digits) of the kernel source each workload runs, as code (comments and blank lines do not count). A run whose
# kernel source differs reports `traffic: null` and says why, so that a change which re-reads data cannot keep
# printing an old ratio.
TRAFFIC_MEASURED_AT = {"pagecopy_kernels.hip": "f06fe4ee28b950af", "transpose_kernels.hip": "a4148a94bb8dc054"}


def kernel_source_digest(fname):
    import hashlib
    import re
    h = hashlib.sha256()
    with open(os.path.join(ROOT, "bi-kv_amd", "csrc", fname)) as fh:
        for line in fh:
            code = re.sub(r"//.*$", "", line).strip()
            if code:
                h.update(code.encode() + b"\n")
    return h.hexdigest()[:16]


def traffic_ratio(workload, kind):
    """(ratio or None, source text) for `traffic` of the dominant kernel."""
    r = MEASURED_TRAFFIC_RATIO.get(workload, {}).get(kind)
    if r is None:
        return None, None
    fname = "transpose_kernels.hip" if workload == "layout_change" else "pagecopy_kernels.hip"
    now = kernel_source_digest(fname)
    if now != TRAFFIC_MEASURED_AT[fname]:
        return None, (f"not reported: {fname} (digest {now}) is not the source the counters under profiles/ were "
                      f"read from (digest {TRAFFIC_MEASURED_AT[fname]})")
    return r, TRAFFIC_SOURCE


def counter_means(csv_path, counter, dominant_kernel):
    """Mean per dispatch of `counter` in a rocprofv3 counter_collection.csv, for the plain-copy calibration
    kernel ("copy") and for the kernels whose name contains `dominant_kernel` ("dominant"): {key: (dispatches,
    mean)}. A dispatch's rows (one per counter instance) are summed."""
    import csv
    csv.field_size_limit(1 << 30)
    per = {}
    with open(csv_path) as fh:
        for row in csv.DictReader(fh):
            if row["Counter_Name"] != counter:
                continue
            k = "copy" if "bikv::copy_runs_wave_kernel" in row["Kernel_Name"] else (
                "dominant" if dominant_kernel in row["Kernel_Name"] else None)
            if k:
                per.setdefault(k, {}).setdefault(row["Dispatch_Id"], 0.0)
                per[k][row["Dispatch_Id"]] += float(row["Counter_Value"])
    return {k: (len(v), sum(v.values()) / len(v)) for k, v in per.items()}


def traffic_from_counters(fetch, write, alg_bytes, copy_bytes=2 << 30):
    """HBM bytes per launch of the dominant kernel from the two counters' means (counter_means): FETCH_SIZE and
    WRITE_SIZE count KiB in units that differ between the two, so each is scaled by what it reads for the plain
    copy of `copy_bytes` each way. Returns (bytes or None, details)."""
    kib = copy_bytes / 1024.0
    fscale = kib / fetch["copy"][1]
    wscale = kib / write["copy"][1]
    fetched = fetch["dominant"][1] * fscale * 1024
    written = write["dominant"][1] * wscale * 1024
    note = {"dispatches": fetch["dominant"][0],
            "fetch_scale_from_plain_copy": round(fscale, 5), "write_scale_from_plain_copy": round(wscale, 5),
            "fetched_bytes": round(fetched), "written_bytes": round(written),
            "ratio_to_algorithmic": round((fetched + written) / alg_bytes, 4)}
    if not (0.5 < fscale < 4 and 0.5 < wscale < 4 and 0.5 < (fetched + written) / alg_bytes < 3):
        note["skipped"] = "the counters are out of line with the calibration copy"
        return None, note
    return round(fetched + written), note


def measure_traffic_live(workload, dominant_kernel, alg_bytes, limit_s=60):
    """HBM bytes per launch of `dominant_kernel`, measured now: this file is run twice more as a child process
    under `rocprofv3 --pmc` (FETCH_SIZE, then WRITE_SIZE; one counter per run), on the same workload at full size
    with three timed steps. Each counter's mean per dispatch of the kernel is scaled by what the same counter
    reads for the plain 2 GiB copy the child also launches. Returns (bytes or None, dict describing the
    measurement); None whenever anything is missing or out of line, in which case the caller keeps the ratio
    recorded under profiles/. The parent must hold no large device allocation while the children run."""
    import glob
    import shutil
    import subprocess
    import tempfile
    note = {"source": "rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE, one child run of this file each, in this run",
            "kernel": dominant_kernel}
    if not shutil.which("rocprofv3"):
        note["skipped"] = "rocprofv3 is not on PATH"
        return None, note
    if any("rocprof" in os.environ.get(k, "") for k in ("LD_PRELOAD", "ROCP_TOOL_LIBRARIES", "HSA_TOOLS_LIB")):
        note["skipped"] = "this process already runs under a profiler"
        return None, note
    tmp = tempfile.mkdtemp(prefix="bikv_traffic_", dir="/tmp")
    env = dict(os.environ, TMPDIR="/tmp")
    means = {}
    try:
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            d = os.path.join(tmp, counter)
            cmd = ["timeout", "-s", "KILL", str(limit_s), "rocprofv3", "--pmc", counter, "--output-format", "csv",
                   "-d", d, "-o", "c", "--", sys.executable, os.path.abspath(__file__), "--workload", workload,
                   "--steps", "3", "--warmup", "1", "--no-cpu-baseline", "--no-other-layout", "--no-configs",
                   "--no-staging", "--no-live-traffic"]
            t0 = time.time()
            r = subprocess.run(cmd, cwd="/tmp", env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE)
            note[f"{counter}_run_s"] = round(time.time() - t0, 1)
            if r.returncode != 0:
                note["skipped"] = f"the {counter} run ended with status {r.returncode}"
                return None, note
            hits = glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)
            if not hits:
                note["skipped"] = f"the {counter} run left no counter file"
                return None, note
            means[counter] = counter_means(hits[0], counter, dominant_kernel)
            if "copy" not in means[counter] or "dominant" not in means[counter]:
                note["skipped"] = f"the {counter} run holds no dispatch of the calibration copy or of {dominant_kernel}"
                return None, note
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    live, details = traffic_from_counters(means["FETCH_SIZE"], means["WRITE_SIZE"], alg_bytes)
    note.update(details)
    return live, note


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="qwen2_7b")
    ap.add_argument("--layout", default="layer_major", choices=["layer_major", "page_major"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-layout", dest="no_other_layout", action="store_true",
                    help="skip the second measurement with the other staging layout")
    ap.add_argument("--pool-form", dest="pool_form", choices=["planar", "worker"], default="planar",
                    help="planar: one [pages, tile] plane per (layer, K|V); worker: one [tokens, 2, heads, dim] tensor per "
                         "layer with K and V interleaved token by token, as the reference's Worker holds its cache")
    ap.add_argument("--pool-pages", type=int, default=0, help="override the pool size (pages per plane)")
    ap.add_argument("--pool-alloc", choices=["planes", "stacked", "spread"], default="spread",
                    help="one torch tensor per (layer, K|V) plane, one stacked torch allocation, or one allocation "
                         "from bikv_device_alloc (physical chunks alternating between the two halves of HBM)")
    ap.add_argument("--staging-alloc", dest="staging_alloc", choices=["torch", "spread", "auto"], default="auto",
                    help="where the dense staging buffers come from: torch, bikv_device_alloc, or auto = the buffer a "
                         "gather WRITES from bikv_device_alloc, the buffer a scatter only reads from torch")
    ap.add_argument("--no-live-traffic", dest="no_live_traffic", action="store_true",
                    help="do not run the two rocprofv3 --pmc child processes that measure the dominant kernel's HBM "
                         "traffic at the end of the default run (roofline.traffic then comes from the recorded ratio)")
    ap.add_argument("--no-configs", dest="no_configs", action="store_true",
                    help="skip the other named configurations (default workload only)")
    ap.add_argument("--no-staging", dest="no_staging", action="store_true",
                    help="skip the pinned-host staging record (default workload only)")
    ap.add_argument("--staging-passes", dest="staging_passes", type=int, default=3)
    ap.add_argument("--staging-requests", dest="staging_requests", type=int, default=128)
    ap.add_argument("--seg", type=int, default=None)
    ap.add_argument("--unroll", type=int, default=None)
    ap.add_argument("--nontemporal", type=int, default=None)
    ap.add_argument("--wave-block", dest="wave_block", type=int, default=None)
    ap.add_argument("--order", type=int, default=None)
    ap.add_argument("--log2-chunk", dest="log2_chunk", type=int, default=None)
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                    help="any launch knob of bikv_set_tuning, e.g. --tune transpose_kvswap=1 (repeatable)")
    ap.add_argument("--staging-cap-gb", dest="staging_cap_gb", type=float, default=32.0,
                    help="largest staging buffer of one launch; bigger batches take several launches")
    ap.add_argument("--chunk-mib", type=int, default=0, help="staging: measure only this chunk size (0 = the sweep)")
    ap.add_argument("--buffers", type=int, default=2, help="staging pipeline lanes with --chunk-mib")
    ap.add_argument("--per-launch", dest="per_launch", type=int, default=4, help="host copies per kernel launch with --chunk-mib")
    return ap.parse_args()


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


ALLOC_NOTES = []   # what happened when memory was asked from bikv_device_alloc (reported in the JSON line)


def spread_empty(bk, nbytes, dev, what):
    """A uint8 device tensor from bikv_device_alloc. If the allocator cannot serve the request (no
    virtual-memory API on this driver, device too full) the measurement still runs, on torch memory, and the
    JSON line says so."""
    import torch
    try:
        buf = bk.DeviceBuffer(nbytes, dev)
        log(f"bikv_device_alloc ({what}): {buf.info}")
        ALLOC_NOTES.append({"what": what, **buf.info})
        return buf.tensor
    except RuntimeError as e:
        log(f"bikv_device_alloc failed for {what}: {e}; using torch memory")
        ALLOC_NOTES.append({"what": what, "failed": str(e)})
        return torch.empty(nbytes, dtype=torch.uint8, device=dev)


def fill_random_bytes(t):
    """Random bytes in place, one plane at a time (bit patterns are what matters for a byte mover)."""
    import torch
    flat = t.view(torch.uint8).reshape(-1)
    step = 1 << 31
    for off in range(0, flat.numel(), step):
        flat[off: off + step].random_(0, 256)


def make_pool(shape, dev, alloc="planes", form="planar"):
    """The pool as the serving engine holds it: one tensor per (layer, K|V) plane ("planes", as
    Bi-KV/Worker/Worker.py:74-78 keeps a list of per-layer caches), or one stacked allocation
    ("stacked"), or memory from bikv_device_alloc ("spread"). Returns (planes, scale planes or None); both
    index as planes[q] -> [n_pages, tile]. With form "worker" the pool is one [tokens, 2, heads, dim] tensor
    per layer (Bi-KV/Worker/Worker.py:74-78); the planes are then strided views [n_pages, page_tokens, row]
    for checking, and the second value is the list of per-layer tensors."""
    import torch

    if form == "worker":
        # [tokens, 2, heads, dim] per layer; plane (l, k) is the strided view [pages, page_tokens, row] of it
        import bikv_pagecopy as bk
        if shape.scales:
            raise SystemExit("bench: the worker form has no scale planes")
        L, P = shape.layers, shape.page_tokens
        row = shape.tile_bytes // P
        n = L * shape.n_pages * P * 2 * row
        arena = spread_empty(bk, n, dev, f"{shape.name} pool, worker form") if alloc == "spread" else \
            torch.empty(n, dtype=torch.uint8, device=dev)
        fill_random_bytes(arena)
        a5 = arena.view(L, shape.n_pages, P, 2, row)
        el = arena.view(torch.float16 if shape.elem_bytes == 2 else torch.uint8)
        layers = list(el.view(L, shape.n_pages * P, 2, shape.kv_heads, shape.head_dim).unbind(0))
        return [a5[l, :, :, k] for l in range(L) for k in (0, 1)], layers

    def one(tile_bytes):
        if alloc == "spread":
            import bikv_pagecopy as bk
            n = shape.n_planes * shape.n_pages * tile_bytes
            t = spread_empty(bk, n, dev, f"{shape.name} pool").view(shape.n_planes, shape.n_pages, tile_bytes)
            fill_random_bytes(t)
            return [t[q] for q in range(shape.n_planes)]
        if alloc == "stacked":
            t = torch.empty((shape.n_planes, shape.n_pages, tile_bytes), dtype=torch.uint8, device=dev)
            fill_random_bytes(t)
            return [t[q] for q in range(shape.n_planes)]
        out = [torch.empty((shape.n_pages, tile_bytes), dtype=torch.uint8, device=dev) for _ in range(shape.n_planes)]
        for t in out:
            fill_random_bytes(t)
        return out

    return one(shape.tile_bytes), (one(shape.scale_tile_bytes) if shape.scales else None)


def verify_on_device(pool_t, staging, batch, requests, n_full=2):
    """Independent check at full size: torch.index_select on the device. EVERY plane of the first
    `n_full` non-empty requests and of the last one, three planes (first, middle, last) of all others.
    Returns (ok, plane-request pairs checked, plane-request pairs in the batch)."""
    import torch
    n_planes = len(pool_t)
    some = sorted({0, n_planes // 2, n_planes - 1})
    nonempty = [r for r, ids in enumerate(requests) if len(ids)]
    full = set(nonempty[:n_full] + nonempty[-1:])
    checked = 0
    for r in nonempty:
        view = batch.request_view(staging, r)
        idt = torch.from_numpy(requests[r]).to(pool_t[0].device)
        for q in (range(n_planes) if r in full else some):
            want = torch.index_select(pool_t[q], 0, idt)
            got = view[q] if batch.layout == "layer_major" else view[:, q]
            if not torch.equal(got.reshape(want.shape), want):
                return False, checked, len(nonempty) * n_planes
            checked += 1
    return True, checked, len(nonempty) * n_planes


def launch_stats(ms, alg_bytes):
    """min / median / p99 / mean of a kernel's launch durations (HIP events around each launch)."""
    import numpy as np
    a = np.sort(np.asarray(ms, dtype=np.float64))
    mean = float(a.mean())
    return {"GBps": round(alg_bytes / (mean * 1e-3) / 1e9, 1), "avg_ms": round(mean, 4),
            "min_ms": round(float(a[0]), 4), "median_ms": round(float(np.median(a)), 4),
            "p99_ms": round(float(a[min(len(a) - 1, int(np.ceil(0.99 * len(a))) - 1)]), 4),
            "max_ms": round(float(a[-1]), 4), "launches_timed": int(len(a)), "alg_bytes": int(alg_bytes)}


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


# Where the `traffic` figures come from: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this file, kept as
# summaries under profiles/. They are NOT measured by the run that prints them (counters need the
# profiler); a run only multiplies its own algorithmic bytes by the ratio recorded there.
TRAFFIC_SOURCE = "profiles/<kernel>_<workload>.md (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of this workload; not measured in this run)"


def run_gather_scatter(args, bk, workloads, dev, with_copy=True, name=None, layout=None, steps=None,
                       warmup=None, target_s=None, keep_pool=False, pool_form=None, reuse=None):
    """One named configuration at full size: pool resident in HBM, one launch per direction (more when the
    staging image would exceed --staging-cap-gb), `steps` timed steps (or as many as fill `target_s`
    seconds). Returns (json fragment, shape, workload, kept) — kept = (pool_t, pool) when keep_pool. `reuse` =
    the kept pool of an earlier call on the same shape (planar, no scale class), taken over instead of
    allocating the same pool once more."""
    import numpy as np
    import torch

    name = name or args.workload
    layout = layout or args.layout
    steps = steps or args.steps
    warmup = args.warmup if warmup is None else warmup
    shape = workloads.SHAPES[name]
    if args.pool_pages:
        shape = shape.scaled(args.pool_pages)
    wl = workloads.named(name, shape)
    log(f"{name}: pool {shape.pool_bytes / 1e9:.2f} GB, tile {shape.tile_bytes} B x {shape.n_planes} planes, layout {layout}")
    pool_form = pool_form or args.pool_form
    if reuse is not None:
        pool_t, pool = reuse
        scale_t = None
    else:
        pool_t, scale_t = make_pool(shape, dev, args.pool_alloc, pool_form)
    if reuse is not None:
        pass
    elif pool_form == "worker":                       # second value = the per-layer tensors, not scale planes
        pool, scale_t = bk.PagedKVPool.from_token_kv_layers(scale_t, shape.page_tokens), None
    else:
        pool = bk.PagedKVPool.from_planes(pool_t, scale_t)

    g_reqs = wl["gather"]
    s_reqs = wl.get("scatter") or []
    if pool_form == "worker" and not s_reqs:
        # the named workload only gathers; the Worker also writes received pages into this pool, so the same
        # request lengths are scattered to fresh unique pages as well
        perm, o = np.random.default_rng(7).permutation(shape.n_pages), 0
        for r in g_reqs:
            s_reqs.append(perm[o: o + len(r)].astype(np.int64))
            o += len(r)

    # A launch covers as many whole requests as fit a staging buffer of --staging-cap-gb; the
    # Qwen2-7B-shaped batch fits in one launch per direction, the 70B-shaped one needs a few.
    def groups_of(reqs, unique=False):
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
        return [(pool.make_batch(g, layout, check_unique=unique), g) for g in out]

    g_groups, s_groups = groups_of(g_reqs), groups_of(s_reqs, unique=True)
    max_slots = max(b.n_slots for b, _ in g_groups + s_groups)
    if args.staging_alloc in ("spread", "auto"):
        g_st = spread_empty(bk, max_slots * shape.tile_bytes, dev, f"{name} gather destination")
    else:
        g_st = torch.empty(max_slots * shape.tile_bytes, dtype=torch.uint8, device=dev)
    g_sc = torch.empty(max_slots * shape.scale_tile_bytes, dtype=torch.uint8, device=dev) if shape.scales else None
    s_st = s_sc = None
    if s_groups:
        s_st = (spread_empty(bk, g_st.numel(), dev, f"{name} scatter source") if args.staging_alloc == "spread"
                else torch.empty_like(g_st))
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

    def step(events=None, first=True):
        # events[0] is recorded for the first step only: a later step starts where the one before it ended
        if events is not None and first:
            events[0].record()
        for b, _ in g_groups:
            pool.gather(b, *views(b, g_st, g_sc))
        if events is not None:
            events[1].record()
        for b, _ in s_groups:
            pool.scatter(b, *views(b, s_st, s_sc))
        if events is not None:
            events[2].record()

    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for _ in range(max(1, warmup)):
        step()
    pool.check()
    warm_step_s = (time.perf_counter() - t0) / max(1, warmup)
    if target_s:
        steps = int(min(4000, max(5, np.ceil(target_s / max(warm_step_s, 1e-5)))))
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for k in range(steps):
        step(evs[k], first=(k == 0))
    torch.cuda.synchronize(dev)
    wall = time.perf_counter() - t0
    pool.check()
    for k in range(1, steps):
        evs[k][0] = evs[k - 1][2]

    # per-launch durations (a direction's launches are back to back between two events)
    g_ms = [e[0].elapsed_time(e[1]) / len(g_groups) for e in evs]
    s_ms = [e[1].elapsed_time(e[2]) / max(1, len(s_groups)) for e in evs]
    ms_per_step = wall * 1e3 / steps
    value = (alg_g + alg_s) / (wall / steps) / 1e9

    # parity at full size, outside the timed region: scattered pages must equal their source, and
    # each gather launch is repeated into a cleared buffer and checked against torch.index_select
    ok, checked, total = True, 0, 0
    for grp, st_all, sc_all, regather in ((s_groups, s_st, s_sc, False), (g_groups, g_st, g_sc, True)):
        for b, reqs in grp:
            st, sc = views(b, st_all, sc_all)
            if regather:
                st.zero_()
                pool.gather(b, st, sc)
                pool.check()
            for tensors, image in ((pool_t, st), (scale_t, sc)):
                if tensors is None:
                    continue
                o, c, t = verify_on_device(tensors, image, b, reqs)
                ok, checked, total = ok and o, checked + c, total + t
    if not ok:
        raise SystemExit("bench: results differ from torch.index_select on the device — not reporting")
    alg_g //= len(g_groups)          # per launch, for the roofline entries below
    alg_s //= max(1, len(s_groups))
    g_stat = launch_stats(g_ms, alg_g)
    s_stat = launch_stats(s_ms, alg_s) if s_groups else None

    copy_gbps, copy_ok = time_plain_copy(bk, dev) if with_copy else (0.0, True)
    if not copy_ok:
        raise SystemExit("bench: plain copy mismatch")

    # the dominant kernel = the instantiation that takes more of the step
    dominant_is_gather = (s_stat is None) or (float(np.sum(g_ms)) >= float(np.sum(s_ms)))
    kname = "bikv::tile_move_wave_kernel<0=gather>" if dominant_is_gather else "bikv::tile_move_wave_kernel<1=scatter>"
    dom = g_stat if dominant_is_gather else s_stat
    ratio, ratio_src = traffic_ratio(name, "gather" if dominant_is_gather else "scatter")
    if args.pool_pages or layout != "layer_major" or pool_form == "worker":
        ratio, ratio_src = None, None                  # measured on the full-size layer-major workload only
    out = {
        "metric": "paged-KV gather/scatter HBM GB/s (% of MI355X peak) + pages/s, bit-exact",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": f"{name}: {shape.layers} layers x K/V, {shape.n_pages} pages x {shape.page_tokens} tok x "
                               f"{shape.kv_heads} heads x {shape.head_dim} {shape.dtype}"
                               f"{' + fp32 scales' if shape.scales else ''}; {len(g_reqs)} gather + {len(s_reqs)} "
                               f"scatter requests, {n_pages} pages/step in {len(g_groups)}+{len(s_groups)} launches, "
                               f"layout {layout}"
                               + ("; pool held as one [tokens, 2, heads, dim] tensor per layer (the reference Worker's form: "
                                  f"a tile is {shape.page_tokens} rows of {shape.tile_bytes // shape.page_tokens} B, two rows apart)"
                                  if pool_form == "worker" else ""),
                   "pool_GB": round(shape.pool_bytes / 1e9, 2), "tile_bytes": shape.tile_bytes,
                   "planes": shape.n_planes,
                   "pool_alloc": ("bikv_device_alloc (physical chunks alternating between the halves of HBM)"
                                  if args.pool_alloc == "spread" else f"torch ({args.pool_alloc})"),
                   "staging_alloc": {"auto": "gather destination from bikv_device_alloc, scatter source from torch",
                                     "spread": "bikv_device_alloc", "torch": "torch"}[args.staging_alloc]},
        "timed_region_s": round(wall, 3),
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "pages_per_s": round(n_pages / (wall / steps), 1),
        "bit_exact": True,
        "bit_exact_coverage": f"torch.index_select on the device over {checked} of {total} (request, plane) images: every "
                              "plane of the first two and the last request of each launch, first/middle/last plane of the rest",
        "roofline": {"bound": "hbm", "kernel": kname, "achieved": dom["GBps"], "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(dom["GBps"] / HBM_PEAK_GBPS, 4),
                     "traffic": (round(ratio * dom["alg_bytes"]) if ratio else None),
                     "traffic_source": ratio_src,
                     "alg_bytes_per_launch": dom["alg_bytes"], "avg_launch_ms": dom["avg_ms"]},
        "kernels": {"gather": g_stat, "scatter": s_stat,
                    "plain_copy_2GiB": ({"GBps": round(copy_gbps, 1)} if with_copy else None)},
    }
    kept = None
    if keep_pool:
        kept = (pool_t, pool)
    del g_st, s_st, g_sc, s_sc
    if not keep_pool:
        pool.close()
        del pool_t, scale_t
    torch.cuda.empty_cache()
    return out, shape, wl, kept


def config_summary(o):
    """The part of a configuration's measurement that goes into the default line's `configs` record."""
    k = o["kernels"]
    frac = lambda st: round(st["GBps"] / HBM_PEAK_GBPS, 4) if st else None
    return {"workload": o["config"]["workload"], "pool_GB": o["config"]["pool_GB"], "value": o["value"], "unit": "GB/s",
            "pct_of_hbm_peak": o["pct_of_hbm_peak"], "pages_per_s": o["pages_per_s"], "steps": o["steps"],
            "timed_region_s": o["timed_region_s"], "bit_exact": o["bit_exact"],
            "gather": dict(k["gather"], frac=frac(k["gather"])),
            "scatter": (dict(k["scatter"], frac=frac(k["scatter"])) if k["scatter"] else None),
            "traffic": o["roofline"]["traffic"]}


def link_yardstick(bk, dev, host, dev_buf, reps=3):
    """Plain hipMemcpyAsync of one large pinned buffer, both directions: best of `reps`, GB/s."""
    n = min(host.numel(), dev_buf.numel())
    d2h = max(n / bk.measure_d2h(dev, host, dev_buf, 0) / 1e9 for _ in range(reps))
    h2d = max(n / bk.measure_h2d(dev, dev_buf, host, 0) / 1e9 for _ in range(reps))
    return d2h, h2d


def run_staging(args, bk, workloads, dev, kept=None):
    """Llama-3-8B shape: every request of the log-normal stream gathered into pinned host memory, and
    scattered back from it, through the staging pipeline. All requests of a pass are enqueued back to back
    (one wait at the end). The record has two parts, in the order they are measured:

    first_pass  the first pass of a fresh stager in every mode, taken the moment the pool is ready — no
                warm-up of any kind, with the mean rate of plain 64 MiB hipMemcpyAsync calls right before and
                after it;
    cells       chunk sizes, lane counts and modes, three timed passes each after two untimed ones, each next
                to a plain hipMemcpyAsync of one 1 GiB pinned buffer timed immediately before it. Before the
                first cell the run repeats short pipelined passes until two in a row are at full rate (the
                rates seen and the time are reported): this benchmark has just released hundreds of GB of
                device memory, and for as long as the driver scrubs released memory, copies that land on the
                copy engine it uses run at half rate."""
    import numpy as np
    import torch

    shape = workloads.SHAPES["llama3_8b"]
    if args.pool_pages:
        shape = shape.scaled(args.pool_pages)
    wl = workloads.named("llama3_8b", shape)
    if kept is None:
        pool_t, _ = make_pool(shape, dev, args.pool_alloc)
        pool = bk.PagedKVPool.from_planes(pool_t)
    else:
        pool_t, pool = kept
    reqs = wl["gather"][: max(1, args.staging_requests)]
    layout = "layer_major"
    sizes = np.array([len(r) * shape.page_bytes for r in reqs], dtype=np.int64)
    region = int(max(4 << 30, 2 * sizes.max()))
    host = bk.pinned_empty(region)
    dev_buf = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    # every request gets a window of the pinned region; windows rotate through it, so requests in flight
    # together (neighbours in issue order) never share host bytes
    offs, cur = [], 0
    for sz in sizes:
        if cur + sz > region:
            cur = 0
        offs.append(cur)
        cur += int(sz)
    g_batches = [pool.make_batch([r], layout) for r in reqs]
    # the way back: each image into the pages next to the ones it came from (unique within a request)
    s_batches = [pool.make_batch([(np.asarray(r) + 1) % shape.n_pages], layout, check_unique=True) for r in reqs]
    torch.cuda.synchronize(dev)
    total_bytes = int(sizes.sum())
    passes = max(1, args.staging_passes)
    yard = {"d2h": [], "h2d": []}
    # a prefix of the stream of about 10 GB: what the first-pass and scrub measurements move
    n_short = int(np.searchsorted(np.cumsum(sizes), 10e9)) + 1
    short_bytes = int(sizes[:n_short].sum())

    def one_pass(stager, mode, direction, n_req=None, synchronous=False):
        n_req = len(reqs) if n_req is None else n_req
        batches = g_batches if direction == "gather" else s_batches
        t0 = time.perf_counter()
        for b, off, sz in list(zip(batches, offs, sizes))[:n_req]:
            win = host[off: off + int(sz)]
            if synchronous:
                (stager.gather_to_host if direction == "gather" else stager.scatter_from_host)(pool, b, win, mode)
            else:
                (stager.gather_to_host_async if direction == "gather" else stager.scatter_from_host_async)(pool, b, win, mode)
        if not synchronous:
            stager.wait()
        return int(sizes[:n_req].sum()) / (time.perf_counter() - t0) / 1e9

    def small_copy_rate(direction, seconds=0.15):
        """Mean rate of back-to-back plain hipMemcpyAsync calls of 64 MiB over about `seconds`: the probe that
        tells whether the copy engines are at full rate."""
        n, moved, t0 = 64 << 20, 0, time.perf_counter()
        spent = 0.0
        while True:
            if direction == "d2h":
                spent += bk.measure_d2h(dev, host[:n], dev_buf[:n], 0)
            else:
                spent += bk.measure_h2d(dev, dev_buf[:n], host[:n], 0)
            moved += n
            if time.perf_counter() - t0 >= seconds:
                return moved / spent / 1e9

    def cell(stager, mode, direction, synchronous=False):
        d2h, h2d = link_yardstick(bk, dev, host[: dev_buf.numel()], dev_buf)
        yard["d2h"].append(d2h)
        yard["h2d"].append(h2d)
        link = d2h if direction == "gather" else h2d
        rates = [one_pass(stager, mode, direction, synchronous=synchronous) for _ in range(passes + 2)][2:]
        return {"GBps_min": round(min(rates), 2), "GBps_median": round(float(np.median(rates)), 2),
                "plain_GBps_just_before": round(link, 2),
                "frac_min": round(min(rates) / link, 4), "frac_median": round(float(np.median(rates)) / link, 4),
                "passes_GBps": [round(r, 2) for r in rates]}

    def verify(stager, mode):
        """Three requests (smallest, median, largest below 1 GiB) staged synchronously and compared, every
        plane, with torch.index_select on the device; then scattered back and read from the pool."""
        order = np.argsort(sizes)
        small = [i for i in order if sizes[i] <= (1 << 30)]
        for i in {int(order[0]), int(order[len(order) // 2]), int(small[-1])}:
            r, b, sz = reqs[i], g_batches[i], int(sizes[i])
            win = host[:sz]
            win.zero_()
            stager.gather_to_host(pool, b, win, mode)
            idt = torch.from_numpy(np.asarray(r)).to(dev)
            view = win.view(shape.n_planes, len(r), shape.tile_bytes)
            for q in range(shape.n_planes):
                if not torch.equal(view[q], torch.index_select(pool_t[q], 0, idt).cpu()):
                    raise SystemExit(f"bench: staged bytes differ ({mode}, request {i}, plane {q})")
            stager.scatter_from_host(pool, s_batches[i], win, mode)
            idt2 = (idt + 1) % shape.n_pages
            for q in (0, shape.n_planes // 2, shape.n_planes - 1):
                if not torch.equal(torch.index_select(pool_t[q], 0, idt2).cpu(), view[q]):
                    raise SystemExit(f"bench: scattered bytes differ ({mode}, request {i}, plane {q})")

    MODES = ("auto", "pipelined_kernel", "pipelined")

    def sweep_modes():
        """One pass of ~10 GB per mode and direction, each in a stager created for it, with the rate of small
        plain copies taken right before and after (are the copy engines at full rate?)."""
        rec = {}
        for direction, probe in (("gather", "d2h"), ("scatter", "h2d")):
            for mode in MODES:
                st = bk.HostStager(dev)
                before = small_copy_rate(probe, 0.05)
                r = one_pass(st, mode, direction, n_short)
                after = small_copy_rate(probe, 0.05)
                st.close()
                rec[f"{direction}_{mode}"] = {"GBps": round(r, 2), "plain_64MiB_copies_before_GBps": round(before, 2),
                                              "plain_64MiB_copies_after_GBps": round(after, 2)}
        return rec

    # --- 1. first pass of every mode, no warm-up, in whatever state this process is in
    t_part = time.perf_counter()
    first = sweep_modes()
    first["what"] = (f"first pass of a fresh stager per mode (library defaults: 16 MiB x 2 copies per launch x 2 lanes), "
                     f"{n_short} requests = {short_bytes / 1e9:.1f} GB, no warm-up of any kind; 'plain' = back-to-back "
                     "hipMemcpyAsync calls of 64 MiB right before / after the pass")
    log(f"staging first_pass {first}")

    # --- 2. wait until the hipMemcpyAsync lanes are back at full rate (the scrub of what this run released), then
    # the cells. The probe is the thing itself: short passes of the pipelined mode on a stager of the default
    # shape (a single plain copy is no probe: in this process it keeps its full rate while the lanes do not).
    t_wait, settle = time.perf_counter(), []
    probe = bk.HostStager(dev)
    plain_now = small_copy_rate("d2h", 0.1)
    while True:
        settle.append(round(one_pass(probe, "pipelined", "gather", n_short), 1))
        if (len(settle) >= 2 and min(settle[-2:]) > 0.93 * plain_now) or time.perf_counter() - t_wait > 60.0:
            break
    probe.close()
    settle_s = time.perf_counter() - t_wait
    # the first DMA into a pinned page is slower than later ones: the whole region has been touched by now
    # only if the passes above covered it, so touch it once
    for off in range(0, region, dev_buf.numel()):
        n = min(dev_buf.numel(), region - off)
        host[off: off + n].copy_(dev_buf[:n])
    if args.chunk_mib:
        grid = [(args.chunk_mib, args.buffers, args.per_launch)]
    else:
        # (chunk MiB, lanes, host copies per kernel launch). The cells proper run on two lanes, the library's
        # default. The rest are contrast cases: more lanes — hipMemcpyAsync on three or four streams at once falls,
        # for whole passes and depending on nothing the library controls, into states where the link moves 37-45
        # GB/s instead of 56 (a process also has only four hardware queues, so a fourth lane runs in turn with
        # the third) — and one kernel per small copy, the shape that made small chunks slow and erratic
        grid = [(4, 2, 4), (8, 2, 4), (16, 2, 2), (32, 2, 1), (4, 3, 4), (16, 3, 1), (4, 4, 4), (16, 4, 1), (4, 4, 1)]
    cells = []
    for chunk, lanes, group in grid:
        stager = bk.HostStager(dev, chunk_bytes=chunk << 20, n_buffers=lanes, chunks_per_launch=group)
        if (chunk, lanes, group) == grid[0]:
            verify(stager, "pipelined")
            verify(stager, "pipelined_kernel")
        row = {"mode": "pipelined", "chunk_MiB": chunk, "lanes": lanes, "copies_per_launch": group}
        if group == 1 and chunk < 16:
            row["contrast_case"] = "one kernel per small copy: the shape that makes small chunks slow, shown for contrast only"
        elif lanes >= 3:
            row["contrast_case"] = ("more lanes than the default two: hipMemcpyAsync on three or four streams at once has whole "
                                    "passes at 37-45 GB/s, in a pattern the library does not control (and a fourth lane shares a "
                                    "hardware queue with the third); shown for contrast only")
        row["gather_to_host"] = cell(stager, "pipelined", "gather")
        row["scatter_from_host"] = cell(stager, "pipelined", "scatter")
        log(f"staging {row}")
        cells.append(row)
        stager.close()
    stager = bk.HostStager(dev)          # the library's defaults: 16 MiB x 2 per launch x 2 lanes
    verify(stager, "direct")
    for mode in ("pipelined_kernel", "direct", "auto"):
        row = {"mode": mode, "chunk_MiB": stager.chunk_bytes >> 20, "lanes": stager.n_buffers,
               "copies_per_launch": stager.chunks_per_launch}
        row["gather_to_host"] = cell(stager, mode, "gather")
        row["scatter_from_host"] = cell(stager, mode, "scatter")
        log(f"staging {row}")
        cells.append(row)
    # what one blocking call per request (the reference's calling pattern, kvcache.py:219-225) costs
    per_call = {"mode": "auto", "one_blocking_call_per_request": True,
                "gather_to_host": cell(stager, "auto", "gather", synchronous=True),
                "scatter_from_host": cell(stager, "auto", "scatter", synchronous=True)}
    stager.close()
    auto = cells[-1]

    out = {"workload": f"llama3_8b: {shape.n_pages} pages x {shape.n_planes} planes x {shape.tile_bytes} B, "
                       f"{len(reqs)} requests of {int(sizes.min() // shape.page_bytes)}..{int(sizes.max() // shape.page_bytes)} "
                       f"pages ({total_bytes / 1e9:.2f} GB per pass), enqueued back to back, {passes} timed passes per cell after two untimed ones",
           "pool_GB": round(shape.pool_bytes / 1e9, 2),
           "first_pass": first,
           "wait_for_full_rate_copies": {"seconds": round(settle_s, 2), "pipelined_pass_GBps_seen": settle,
                                         "what": f"passes of {short_bytes / 1e9:.1f} GB in the pipelined mode (16 MiB x 2 x 2 lanes) from "
                                                 "the end of the first passes until two in a row exceed 93 % of a plain copy (60 s at "
                                                 "most): how long the driver was still scrubbing the device memory this run had released"},
           "plain_d2h_GBps": {"min": round(min(yard["d2h"]), 2), "median": round(float(np.median(yard["d2h"])), 2),
                              "max": round(max(yard["d2h"]), 2), "samples": len(yard["d2h"])},
           "plain_h2d_GBps": {"min": round(min(yard["h2d"]), 2), "median": round(float(np.median(yard["h2d"])), 2),
                              "max": round(max(yard["h2d"]), 2), "samples": len(yard["h2d"])},
           "host_link_GBps": auto["gather_to_host"]["GBps_median"],
           "frac_of_plain_d2h": auto["gather_to_host"]["frac_median"],
           "frac_of_best_plain_d2h_seen": round(auto["gather_to_host"]["GBps_median"] / max(yard["d2h"]), 4),
           "scatter_from_host_GBps": auto["scatter_from_host"]["GBps_median"],
           "scatter_frac_of_plain_h2d": auto["scatter_from_host"]["frac_median"],
           "cells": cells, "per_request_blocking_calls": per_call, "bit_exact": True,
           "seconds": round(time.perf_counter() - t_part, 1)}
    real = [c for c in cells if "contrast_case" not in c]
    out["min_frac_over_cells"] = {
        "gather_to_host": min(c["gather_to_host"]["frac_min"] for c in real),
        "scatter_from_host": min(c["scatter_from_host"]["frac_min"] for c in real),
        "what": "lowest single pass of any cell, as a fraction of the plain copy timed just before that cell "
                "(every chunk size and mode above on two lanes, the library's default; the contrast cases — three and "
                "four lanes, one kernel per small copy — are reported in `cells` and left out here)"}
    worst = min(real, key=lambda c: c["gather_to_host"]["frac_min"])
    out["min_frac_over_cells"]["gather_to_host_worst_cell"] = (f"{worst['mode']} {worst['chunk_MiB']} MiB x {worst['lanes']} lanes x "
                                                               f"{worst['copies_per_launch']} per launch, passes {worst['gather_to_host']['passes_GBps']}")
    out["median_frac_over_cells"] = {
        "gather_to_host": round(float(np.median([c["gather_to_host"]["frac_median"] for c in real])), 4),
        "scatter_from_host": round(float(np.median([c["scatter_from_host"]["frac_median"] for c in real])), 4)}
    if kept is None:
        pool.close()
        del pool_t
        torch.cuda.empty_cache()
    return out


def trace_summary(steps):
    """A stager trace (HostStager.trace_read) reduced to what tells where the time of a pass goes: per kind of
    step the count and duration percentiles; copies by their position behind their lane's last kernel; how much
    of the pass at least one copy was running, how far the lanes' copy intervals overlap, and the gaps between
    consecutive steps of a lane."""
    import numpy as np
    if not steps:
        return None
    span = max(s["end_ms"] for s in steps) - min(s["start_ms"] for s in steps)
    out = {"steps": len(steps), "span_ms": round(span, 2), "kinds": {}, "copies_by_position_behind_their_kernel": {}}
    for kind in sorted({s["kind"] for s in steps}):
        ss = [s for s in steps if s["kind"] == kind]
        d = np.array([s["end_ms"] - s["start_ms"] for s in ss])
        b = float(sum(s["bytes"] for s in ss))
        out["kinds"][kind] = {"n": len(ss), "MiB_per_step": round(b / len(ss) / 2 ** 20, 2), "ms_mean": round(float(d.mean()), 4),
                              "ms_p10": round(float(np.percentile(d, 10)), 4), "ms_p50": round(float(np.percentile(d, 50)), 4),
                              "ms_p90": round(float(np.percentile(d, 90)), 4), "ms_max": round(float(d.max()), 4),
                              "GBps_while_running": round(b / max(float(d.sum()), 1e-9) / 1e6, 1)}
    lanes = sorted({s["lane"] for s in steps})
    pos, gaps = {}, {}
    for lane in lanes:
        ls = [s for s in steps if s["lane"] == lane]
        k = 0
        for s in ls:
            if s["kind"] == "kernel":
                k = 0
            elif s["kind"].startswith("copy"):
                k += 1
                pos.setdefault(k, []).append(s["end_ms"] - s["start_ms"])
        g = np.array([ls[i + 1]["start_ms"] - ls[i]["end_ms"] for i in range(len(ls) - 1)] or [0.0])
        gaps[f"lane_{lane}"] = {"steps": len(ls), "gap_ms_p50": round(float(np.percentile(g, 50)), 4),
                                "gap_ms_p90": round(float(np.percentile(g, 90)), 4), "gap_ms_max": round(float(g.max()), 3)}
    for k in sorted(pos):
        d = np.array(pos[k])
        out["copies_by_position_behind_their_kernel"][f"copy_{k}"] = {
            "n": len(d), "ms_p50": round(float(np.percentile(d, 50)), 4), "ms_p90": round(float(np.percentile(d, 90)), 4)}
    cs = sorted((s["start_ms"], s["end_ms"]) for s in steps if s["kind"].startswith("copy"))
    if cs:
        busy, cur_s, cur_e = 0.0, cs[0][0], cs[0][1]
        for a_, b_ in cs[1:]:
            if a_ > cur_e:
                busy += cur_e - cur_s
                cur_s, cur_e = a_, b_
            else:
                cur_e = max(cur_e, b_)
        busy += cur_e - cur_s
        cb = sum(s["bytes"] for s in steps if s["kind"].startswith("copy"))
        out["copies"] = {"some_copy_running_pct_of_span": round(100 * busy / span, 1),
                         "GBps_while_some_copy_runs": round(cb / busy / 1e6, 1),
                         "overlap_factor": round(sum(e - a_ for a_, e in cs) / busy, 2)}
    out["gaps_between_steps_of_a_lane"] = gaps
    return out


def run_staging_trace(args, bk, workloads, dev):
    """Where the time of a pipelined pass goes, step by step: the library's own trace (two events around every
    kernel launch and host copy of a lane, bikv_stager_trace) of the FIRST pass a fresh process makes and of a
    later one, for the hipMemcpyAsync pipeline and for the copy-kernel pipeline. Llama-3-8B-shaped pool of
    --pool-pages pages (default 8192 = 34 GB), the first --staging-requests requests (default here: 24, 10 GB
    per pass), passes back to back."""
    import numpy as np
    import torch
    shape = workloads.SHAPES["llama3_8b"].scaled(args.pool_pages or 8192)
    wl = workloads.named("llama3_8b", shape)
    pool_t, _ = make_pool(shape, dev, args.pool_alloc)
    pool = bk.PagedKVPool.from_planes(pool_t)
    reqs = wl["gather"][: (args.staging_requests if args.staging_requests != 128 else 24)]
    sizes = np.array([len(r) * shape.page_bytes for r in reqs], dtype=np.int64)
    region = int(max(4 << 30, 2 * sizes.max()))
    host = bk.pinned_empty(region)
    offs, cur = [], 0
    for sz in sizes:
        if cur + sz > region:
            cur = 0
        offs.append(cur)
        cur += int(sz)
    batches = [pool.make_batch([r], "layer_major") for r in reqs]
    total = int(sizes.sum())
    torch.cuda.synchronize(dev)
    t_ready = time.perf_counter()
    chunk, lanes, group = (args.chunk_mib or 16), args.buffers, (args.per_launch if args.chunk_mib else 2)
    record = {"workload": f"llama3_8b x {shape.n_pages} pages, {len(reqs)} requests = {total / 1e9:.1f} GB per pass, "
                          f"{chunk} MiB x {group} copies per launch x {lanes} lanes", "modes": {}}
    def run_passes(st, mode, n, traced=()):
        rates, traces = [], {}
        for p in range(n):
            if p in traced:
                st.trace(40000)
            t0 = time.perf_counter()
            for b, off, sz in zip(batches, offs, sizes):
                st.gather_to_host_async(pool, b, host[off: off + int(sz)], mode)
            st.wait()
            rates.append(round(total / (time.perf_counter() - t0) / 1e9, 1))
            if p in traced:
                traces[f"pass_{p}"] = dict(trace_summary(st.trace_read()), GBps=rates[-1],
                                           started_s_after_setup=round(t0 - t_ready, 2))
                st.trace(0)
        return rates, traces

    dev_buf = torch.empty(64 << 20, dtype=torch.uint8, device=dev)

    def plain(seconds=0.15):
        """mean rate of back-to-back plain hipMemcpyAsync calls of 64 MiB (a fresh stream each)"""
        n, moved, spent, t0 = dev_buf.numel(), 0, 0.0, time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            spent += bk.measure_d2h(dev, host[:n], dev_buf, 0)
            moved += n
        return round(moved / spent / 1e9, 1)

    def fresh():
        return bk.HostStager(dev, chunk_bytes=chunk << 20, n_buffers=lanes, chunks_per_launch=group)

    # 1. the first thing the process stages, right behind the pool's placement (which released its filler chunks)
    for mode in ("pipelined", "pipelined_kernel"):
        st = fresh()
        rates, traces = run_passes(st, mode, 10, traced=(0, 8))
        st.close()
        record["modes"][mode] = {"passes_GBps": rates, "plain_64MiB_d2h_after_GBps": plain(), "traces": traces}
        log(f"staging_trace {mode}: {rates}")
    # 2. nothing released for a while: a fresh stager, first pass traced
    time.sleep(8.0)
    st = fresh()
    rates, traces = run_passes(st, "pipelined", 6, traced=(0,))
    st.close()
    record["settled"] = {"what": "a fresh stager 8 s later, nothing released in between", "plain_64MiB_d2h_before_GBps": plain(),
                         "pipelined_passes_GBps": rates, "traces": traces}
    log(f"staging_trace settled: {rates}")
    # 3. 32 GiB of device memory allocated and released (the release returns at once), then a fresh stager at once
    t_rel = time.perf_counter()
    bk.DeviceBuffer(32 << 30, dev, spread=False).free()
    rel_ms = (time.perf_counter() - t_rel) * 1e3
    before = plain(0.1)
    st = fresh()
    rates, traces = run_passes(st, "pipelined", 14, traced=(0,))
    after = plain()
    k_rates, _ = run_passes(st, "pipelined_kernel", 3)
    st.close()
    bk.DeviceBuffer(32 << 30, dev, spread=False).free()
    st = fresh()
    k2_rates, _ = run_passes(st, "pipelined_kernel", 6)
    d_rates, _ = run_passes(st, "direct", 3)
    st.close()
    record["after_release"] = {"what": "32 GiB allocated and released (bikv_device_alloc sequential + bikv_device_free, "
                                       f"{rel_ms:.0f} ms for both), then a fresh stager at once",
                               "plain_64MiB_d2h_right_after_the_release_GBps": before, "pipelined_passes_GBps": rates,
                               "seconds_per_pass": round(total / 1e9 / max(rates[0], 1e-9), 3),
                               "plain_64MiB_d2h_after_the_passes_GBps": after, "pipelined_kernel_passes_after_GBps": k_rates,
                               "second_release_then_pipelined_kernel_passes_GBps": k2_rates, "then_direct_passes_GBps": d_rates,
                               "traces": traces}
    log(f"staging_trace after release: {rates} | kernel hop right after a second release: {k2_rates}")
    pool.close()
    return record


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


def run_reference_ipc(dev, transfers=10):
    """The reference's own scenario through its own operator API, timed the way its script times it
    (Bi-KV/SharedMemory/CUDA_Shared/test_page_ipc.py:41-102,127-162): producer and consumer roles of
    `ipc_service` (here in one process), 200 pages x 50 tokens x (128, 2, 28, 2) fp16 = 273.4 MiB per
    transfer, identity offsets, value 7. One untimed transfer, then `transfers` timed ones: each is one
    blocking producer_copy_pages call (page copy into the ring, stream sync, publication) followed by one
    consumer_receive; the producer's and the consumer's "Throughput" are the script's own formulas (MiB of
    one transfer / mean call time). Beside it the same transfer on the reference's CPU path: torch.index_select
    of the 200 page rows of a host tensor into a host buffer."""
    import torch
    import ipc_service

    page_size, num_pages, head, kvh, layers, kv = 50, 200, 128, 2, 28, 2
    page_elements = page_size * head * kvh * layers * kv
    name = f"/bikv_bench_{os.getpid()}"
    ipc_service.producer_cleanup()
    ipc_service.consumer_cleanup()
    ipc_service.consumer_init(0, name, (2 << 30) - 4096)     # the script's ring is 2 GiB; one that size is not exported over IPC
    ipc_service.producer_init(0, name)
    try:
        cache = torch.full((num_pages, page_size, head, kvh, layers, kv), 7, dtype=torch.float16, device=dev)
        offs = torch.arange(num_pages, dtype=torch.int64, device=dev) * page_elements
        dims = ipc_service.TensorDims()
        dims.total_tokens, dims.head_size, dims.num_kv_heads, dims.num_layers, dims.kv_pair = num_pages * page_size, head, kvh, layers, kv
        torch.cuda.synchronize(dev)
        prod, cons, result = [], [], None
        for i in range(transfers + 1):
            t0 = time.perf_counter()
            ipc_service.producer_copy_pages(cache, offs, offs, page_size, dims)
            t1 = time.perf_counter()
            result = ipc_service.consumer_receive()
            t2 = time.perf_counter()
            if tuple(result.shape) != (num_pages * page_size, head, kvh, layers, kv):
                raise SystemExit(f"bench: reference scenario published shape {tuple(result.shape)}")
            if i:
                prod.append(t1 - t0)
                cons.append(t2 - t1)
        if not bool((result == 7).all().item()):
            raise SystemExit("bench: reference scenario data corrupted")
        mib = cache.numel() * cache.element_size() / (1024 ** 2)
    finally:
        ipc_service.producer_cleanup()
        ipc_service.consumer_cleanup()
    # CPU twin: the same 200 page rows selected out of a host tensor
    host = torch.full((num_pages, page_elements), 7, dtype=torch.float16)
    out = torch.empty_like(host)
    ids = torch.arange(num_pages, dtype=torch.int64)
    cpu = []
    for i in range(transfers + 1):
        t0 = time.perf_counter()
        torch.index_select(host, 0, ids, out=out)
        if i:
            cpu.append(time.perf_counter() - t0)
    avg_p, avg_c = sum(prod) / len(prod), sum(cpu) / len(cpu)
    return {"workload": "reference_200x50 through ipc_service.producer_copy_pages -> ring -> consumer_receive "
                        "(test_page_ipc.py), one process, 1 untimed + %d timed transfers" % transfers,
            "MiB_per_transfer": round(mib, 2),
            "producer_avg_transfer_ms": round(avg_p * 1e3, 4), "producer_MiB_per_s": round(mib / avg_p, 1),
            "consumer_avg_receive_ms": round(sum(cons) / len(cons) * 1e3, 4),
            "consumer_MiB_per_s": round(mib * len(cons) / sum(cons), 1),
            "HBM_GBps_read_plus_written": round(2 * mib * 1024 ** 2 / avg_p / 1e9, 1),
            "cpu_index_select": {"avg_transfer_ms": round(avg_c * 1e3, 3), "MiB_per_s": round(mib / avg_c, 1),
                                 "cores": torch.get_num_threads(), "kind": "port"},
            "bit_exact": True}


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
    g_ids = np.concatenate(wl["gather"]).astype(np.int64)
    s_ids = np.concatenate(wl["scatter"]).astype(np.int64)
    n_g, n_s = len(g_ids), len(s_ids)
    if args.pool_alloc == "spread":
        pool = spread_empty(bk, shape.n_pages * page_elems * 2, dev, "token-major pool").view(torch.bfloat16)
    else:
        pool = torch.empty(shape.n_pages * page_elems, dtype=torch.bfloat16, device=dev)
    fill_random_bytes(pool)
    if args.staging_alloc in ("auto", "spread"):     # the gather writes it, the scatter reads it
        dense = spread_empty(bk, max(n_g, n_s) * page_elems * 2, dev, "dense buffer").view(torch.bfloat16)
    else:
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
                   "pool_GB": round(shape.pool_bytes / 1e9, 2),
                   "pool_alloc": "bikv_device_alloc" if args.pool_alloc == "spread" else "torch"},
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "pages_per_s": round((n_g + n_s) / (wall / args.steps), 1), "bit_exact": True,
        "kernels": {"gather": {"GBps": round(alg_g / g_ms / 1e6, 1), "avg_ms": round(g_ms, 4), "alg_bytes": alg_g},
                    "scatter": {"GBps": round(alg_s / s_ms / 1e6, 1), "avg_ms": round(s_ms, 4), "alg_bytes": alg_s}},
        "roofline": {"bound": "hbm", "kernel": "bikv::copy_runs_wave_kernel", "achieved": round(alg / ms / 1e6, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(alg / ms / 1e6 / HBM_PEAK_GBPS, 4),
                     "traffic": (int(alg * traffic_ratio("qwen2_7b_token_major", "gather" if slow_g else "scatter")[0])
                                 if not args.pool_pages and traffic_ratio("qwen2_7b_token_major", "gather")[0] else None),
                     "alg_bytes_per_launch": alg, "avg_launch_ms": round(ms, 4)},
    }


def run_layout_change(args, bk, dev, blocks=None, sort=False, pool_alloc=None):
    """Received token-major pages -> the Worker's per-layer paged pool and back, at the reference's own
    shapes: token_shape (128, 2, 28, 2) fp16 (Model/qwen2.py:512-522), 28 layer tensors of
    [blocks*16, 2, 2, 128] (Worker.py:69-78: 10240 blocks), 4096 pages of 16 tokens per step and
    direction, random blocks. The pool's memory comes from bikv_device_alloc (`--pool-alloc spread`, the
    default) or from torch. The page lists are built on the host and handed over through NHDPool.page_list;
    with `sort` the load walks its list in ascending block order (worth ~4 % on a torch-allocated pool that
    sits in one half of HBM, nothing on a spread pool)."""
    import numpy as np
    import torch
    from oracle import pagecopy_oracle as oracle

    P, D, H, L, n_pages = 16, 128, 2, 28, 4096
    blocks = blocks or args.pool_pages or 10240
    n_pages = min(n_pages, blocks)
    pool_alloc = pool_alloc or args.pool_alloc
    if pool_alloc == "spread":
        arena = spread_empty(bk, L * blocks * P * 2 * H * D * 2, dev, "layer tensors")
        layers = list(arena.view(torch.float16).view(L, blocks * P, 2, H, D).unbind(0))
    elif pool_alloc == "placed_torch":
        # the reference's own allocation code (one torch tensor per layer), inside the library's torch memory pool
        with bk.placed_allocations(dev):
            layers = [torch.empty((blocks * P, 2, H, D), dtype=torch.float16, device=dev) for _ in range(L)]
    else:
        layers = [torch.empty((blocks * P, 2, H, D), dtype=torch.float16, device=dev) for _ in range(L)]
    for t in layers:
        fill_random_bytes(t)
    pool = bk.NHDPool.from_token_kv_layers(layers, P)
    tm = torch.empty((n_pages, P, D, H, L, 2), dtype=torch.float16, device=dev)
    fill_random_bytes(tm)
    if pool_alloc in ("spread", "placed_torch") and args.staging_alloc in ("auto", "spread"):   # the written image, like a gather's
        tm_out = spread_empty(bk, tm.numel() * 2, dev, "token-major image written by the store").view(torch.float16).view(tm.shape)
    else:
        tm_out = torch.empty_like(tm)
    rng = np.random.default_rng(6)
    ids_h = rng.permutation(blocks)[:n_pages].astype(np.int64)       # page i of tm <-> block ids_h[i]
    ids, pages = pool.page_list(ids_h, sort=sort, check_unique=True)
    ids_s, pages_s = pool.page_list(ids_h, sort=False)
    alg = 2 * tm.numel() * 2                       # bytes read + written per launch

    def step(ev=None):
        if ev:
            ev[0].record()
        pool.load_token_major(tm, ids, pages)      # received pages -> pool blocks
        if ev:
            ev[1].record()
        pool.store_token_major(tm_out, ids_s, pages_s)  # the same blocks -> pages to send
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
    # a sample of pages against the CPU oracle (np.zeros is lazily backed: only the sampled blocks are touched)
    sample = np.arange(0, n_pages, max(1, n_pages // 8))[:8]
    lay_h = [np.zeros((blocks * P, 2, H, D), dtype=np.uint16) for _ in range(L)]
    tm_h = tm[torch.from_numpy(sample).to(dev)].cpu().view(torch.int16).numpy().view(np.uint16)
    oracle.transpose_pages_c(lay_h, "token_kv", np.ascontiguousarray(tm_h), ids_h[sample], np.arange(len(sample)), "load")
    for l in (0, L // 2, L - 1):
        for b in ids_h[sample]:
            got = layers[l][b * P:(b + 1) * P].cpu().view(torch.int16).numpy().view(np.uint16)
            if got.tobytes() != lay_h[l][b * P:(b + 1) * P].tobytes():
                raise SystemExit("bench: layout change differs from the oracle")
    l_stat = launch_stats([e[0].elapsed_time(e[1]) for e in evs], alg)
    s_stat = launch_stats([e[1].elapsed_time(e[2]) for e in evs], alg)
    slow_is_load = l_stat["avg_ms"] >= s_stat["avg_ms"]
    dom = l_stat if slow_is_load else s_stat
    at_reference_shape = blocks == 10240 and pool_alloc == "spread"
    out = {
        "metric": "paged-KV gather/scatter HBM GB/s (% of MI355X peak) + pages/s, bit-exact",
        "value": round(2 * alg / (wall / args.steps) / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall * 1e3 / args.steps, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u16", "data": "synthetic",
        "config": {"workload": f"layout_change: token-major pages <-> {L} layer tensors [{blocks}*{P}, 2, {H}, {D}] fp16, "
                               f"{n_pages} pages of {P} tokens loaded then stored per step, random blocks"
                               f"{'; the load walks them in ascending block order' if sort else ''}",
                   "pool_GB": round(L * blocks * P * 2 * H * D * 2 / 1e9, 2),
                   "pool_alloc": {"spread": "bikv_device_alloc (chunks alternating between the halves of HBM)",
                                  "placed_torch": "28 torch.empty calls inside bikv_pagecopy.placed_allocations()"}.get(pool_alloc, "torch")},
        "timed_region_s": round(wall, 3),
        "pct_of_hbm_peak": round(100 * 2 * alg / (wall / args.steps) / 1e9 / HBM_PEAK_GBPS, 2),
        "pages_per_s": round(2 * n_pages / (wall / args.steps), 1), "bit_exact": True,
        "roofline": {"bound": "hbm", "kernel": f"bikv::transpose_pairs_kernel<{1 if slow_is_load else 0}, 2, 512>",
                     "achieved": dom["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(dom["GBps"] / HBM_PEAK_GBPS, 4),
                     "traffic": (int(alg * traffic_ratio("layout_change", "load" if slow_is_load else "store")[0])
                                 if at_reference_shape and traffic_ratio("layout_change", "load")[0] else None),
                     "traffic_source": traffic_ratio("layout_change", "load")[1] if at_reference_shape else None,
                     "alg_bytes_per_launch": alg, "avg_launch_ms": dom["avg_ms"]},
        "kernels": {"load": l_stat, "store": s_stat},
    }
    pool.close()
    del layers, tm, tm_out
    torch.cuda.empty_cache()
    return out


def emit(out):
    if ALLOC_NOTES:
        out["device_alloc"] = ALLOC_NOTES
    if "summary" in out:
        out["summary"] = out.pop("summary")      # keeps it the last key of the line
    print(json.dumps(out), flush=True)


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
    for kv in args.tune:
        k, _, v = kv.partition("=")
        knobs[k.strip()] = int(v)
    if knobs:
        bk.set_tuning(**knobs)

    if args.workload == "reference_200x50":
        out = run_reference_scenario(args, bk, dev)
        emit(out)
        return
    if args.workload == "qwen2_7b_token_major":
        out = run_token_major(args, bk, workloads, dev)
        emit(out)
        return
    if args.workload == "layout_change":
        # the reference's pool (10240 blocks per layer, 4.7 GB); then the same step on a torch-allocated pool
        # (wherever the driver puts it), that pool with the load's page list sorted by block, and a pool that
        # fills a production share of HBM (163840 blocks, 75 GB)
        out = run_layout_change(args, bk, dev)
        if not args.pool_pages:
            for key, kw in (("torch_alloc", dict(pool_alloc="stacked")), ("torch_alloc_sorted_load", dict(pool_alloc="stacked", sort=True)),
                            ("torch_alloc_inside_placed_allocations", dict(pool_alloc="placed_torch")),
                            ("pool_163840_blocks", dict(blocks=163840))):
                o = run_layout_change(args, bk, dev, **kw)
                out[key] = {"workload": o["config"]["workload"], "pool_GB": o["config"]["pool_GB"], "value": o["value"],
                            "pct_of_hbm_peak": o["pct_of_hbm_peak"], "kernels": o["kernels"]}
        emit(out)
        return
    if args.workload == "staging_trace":
        print(json.dumps({"metric": "pinned-host staging GB/s", "unit": "GB/s", "n_gpus": 1,
                          "staging_trace": run_staging_trace(args, bk, workloads, dev), "device_alloc": ALLOC_NOTES}), flush=True)
        return
    if args.workload == "staging":
        print(json.dumps({"metric": "pinned-host staging GB/s", "unit": "GB/s", "n_gpus": 1,
                          "staging": run_staging(args, bk, workloads, dev)}), flush=True)
        return
    same_pool_again = not args.no_other_layout and args.pool_form == "planar" and not workloads.SHAPES[args.workload].scales
    out, shape, wl, kept = run_gather_scatter(args, bk, workloads, dev, keep_pool=same_pool_again)
    if knobs:
        out["config"]["tuning"] = knobs
    if not args.no_other_layout:
        # the same request stream with the other staging image (reported next to the headline number), on
        # the same pool where that is possible
        alt_layout = "page_major" if args.layout == "layer_major" else "layer_major"
        log(f"same workload, staging layout {alt_layout}")
        o2, _, _, _ = run_gather_scatter(args, bk, workloads, dev, with_copy=False, layout=alt_layout, target_s=0.6, warmup=3,
                                         reuse=kept)
        kept = None
        out["other_layout"] = {"layout": alt_layout, "value": o2["value"], "pct_of_hbm_peak": o2["pct_of_hbm_peak"],
                               "steps": o2["steps"], "kernels": {k: v for k, v in o2["kernels"].items() if v}}
    default_run = args.workload == "qwen2_7b" and not args.pool_pages
    if default_run and args.pool_alloc == "spread" and not args.no_other_layout:
        # the same workload with pool and staging from torch.empty (hipMalloc), wherever the driver places them
        import copy
        alt = copy.copy(args)
        alt.pool_alloc, alt.staging_alloc = "stacked", "torch"
        log("same workload, pool and staging allocated by torch")
        o3, _, _, _ = run_gather_scatter(alt, bk, workloads, dev, with_copy=False, target_s=0.6, warmup=3)
        out["torch_alloc"] = {"value": o3["value"], "pct_of_hbm_peak": o3["pct_of_hbm_peak"], "steps": o3["steps"],
                              "kernels": {k: v for k, v in o3["kernels"].items() if v}}
    if default_run and not args.no_configs:
        # the other named configurations, each at full size: allocated, measured for about a second, freed
        out["configs"] = {}
        for other in ("qwen2_1p5b", "llama3_8b", "llama3_70b_fp8"):
            keep = other == "llama3_8b" and not args.no_staging
            o, _, _, kept = run_gather_scatter(args, bk, workloads, dev, with_copy=False, name=other, target_s=1.0,
                                               warmup=3, keep_pool=keep)
            out["configs"][other] = config_summary(o)
            if other == "qwen2_1p5b":
                # the same shape held the way the reference's Worker holds it: [tokens, 2, heads, dim] per layer
                o, _, _, _ = run_gather_scatter(args, bk, workloads, dev, with_copy=False, name=other, target_s=0.6,
                                                warmup=3, pool_form="worker")
                out["configs"]["qwen2_1p5b_worker_form"] = config_summary(o)
            if keep:
                log("pinned-host staging on the Llama-3-8B pool")
                out["staging"] = run_staging(args, bk, workloads, dev, kept)
                kept[1].close()
                del kept
                torch.cuda.empty_cache()
    elif args.workload == "llama3_8b" and not args.no_staging:
        out["staging"] = run_staging(args, bk, workloads, dev)
    if default_run and not args.no_configs:
        # the layout change at the reference's own shape (28 layer tensors [10240*16, 2, 2, 128] fp16), about
        # a quarter of a second of launches, and the reference's scripted scenario through its operator API
        import copy
        lc_args = copy.copy(args)
        lc_args.steps, lc_args.warmup = 200, 5
        o = run_layout_change(lc_args, bk, dev)
        out["layout_change"] = {"workload": o["config"]["workload"], "pool_GB": o["config"]["pool_GB"], "value": o["value"],
                                "pct_of_hbm_peak": o["pct_of_hbm_peak"], "steps": o["steps"], "bit_exact": o["bit_exact"],
                                "kernels": o["kernels"], "traffic": o["roofline"]["traffic"]}
        log("the reference's 200 x 50 scenario through ipc_service")
        out["reference_scenario"] = run_reference_ipc(dev)
    if not args.no_cpu_baseline:
        log("timing the CPU baseline")
        out["cpu_baseline"] = cpu_baseline(shape, wl)
    if default_run and not args.no_live_traffic:
        # the dominant kernel's HBM traffic, measured now (every measurement above is finished and its memory freed)
        import gc
        gc.collect()
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
        free_b, _ = torch.cuda.mem_get_info()
        rf = out["roofline"]
        if free_b < (150 << 30):
            rf["traffic_live"] = {"skipped": f"only {free_b / 2**30:.0f} GiB of device memory free for the child runs"}
        else:
            log("measuring the dominant kernel's HBM traffic (two rocprofv3 --pmc child runs)")
            dom = "tile_move_wave_kernel<0" if "gather" in rf["kernel"] else "tile_move_wave_kernel<1"
            live, note = measure_traffic_live(args.workload, dom, rf["alg_bytes_per_launch"])
            rf["traffic_live"] = note
            if live is not None:
                rf["traffic_from_recorded_ratio"] = rf["traffic"]
                rf["traffic"] = live
                rf["traffic_source"] = note["source"]
    if default_run:
        add_summary(out)
    emit(out)


def add_summary(out):
    """The figures of the whole run, flat and short, under `config` (and once more as the last key of the line):
    every named configuration's value and per-kernel fraction of 8 TB/s, the torch-allocated headline, the
    staging record's fractions of the plain copy with its first passes, the layout change and the reference's
    scenario. Keys are absent for parts that were skipped."""
    frac = lambda gbps: round(gbps / HBM_PEAK_GBPS, 4)
    sm = {"headline_value_GBps": out["value"],
          "headline_gather_frac": frac(out["kernels"]["gather"]["GBps"]),
          "headline_scatter_frac": frac(out["kernels"]["scatter"]["GBps"]) if out["kernels"]["scatter"] else None}
    rf = out.get("roofline") or {}
    if rf.get("traffic"):
        sm["headline_traffic_over_algorithmic"] = round(rf["traffic"] / rf["alg_bytes_per_launch"], 4)
        sm["headline_traffic_measured_in_this_run"] = "traffic_from_recorded_ratio" in rf
    if "other_layout" in out:
        sm["page_major_value_GBps"] = out["other_layout"]["value"]
    if "torch_alloc" in out:
        sm["torch_alloc_value_GBps"] = out["torch_alloc"]["value"]
        for k, v in out["torch_alloc"]["kernels"].items():
            if k in ("gather", "scatter"):
                sm[f"torch_alloc_{k}_frac"] = frac(v["GBps"])
    for name, c in (out.get("configs") or {}).items():
        sm[f"{name}_value_GBps"] = c["value"]
        sm[f"{name}_gather_frac"] = c["gather"]["frac"]
        if c["scatter"]:
            sm[f"{name}_scatter_frac"] = c["scatter"]["frac"]
    st = out.get("staging")
    if st:
        sm["staging_host_link_GBps"] = st["host_link_GBps"]
        sm["staging_plain_d2h_GBps"] = st["plain_d2h_GBps"]["median"]
        sm["staging_plain_h2d_GBps"] = st["plain_h2d_GBps"]["median"]
        sm["staging_auto_gather_frac_median"] = st["frac_of_plain_d2h"]
        sm["staging_auto_scatter_frac_median"] = st["scatter_frac_of_plain_h2d"]
        sm["staging_gather_frac_min_over_cells"] = st["min_frac_over_cells"]["gather_to_host"]
        sm["staging_scatter_frac_min_over_cells"] = st["min_frac_over_cells"]["scatter_from_host"]
        sm["staging_gather_frac_median_over_cells"] = st["median_frac_over_cells"]["gather_to_host"]
        sm["staging_scatter_frac_median_over_cells"] = st["median_frac_over_cells"]["scatter_from_host"]
        for k, v in st["first_pass"].items():
            if isinstance(v, dict):
                sm[f"staging_first_pass_{k}_GBps"] = v["GBps"]
        sm["staging_wait_for_full_rate_copies_s"] = st["wait_for_full_rate_copies"]["seconds"]
    lc = out.get("layout_change")
    if lc:
        sm["layout_change_value_GBps"] = lc["value"]
        sm["layout_change_load_frac"] = frac(lc["kernels"]["load"]["GBps"])
        sm["layout_change_store_frac"] = frac(lc["kernels"]["store"]["GBps"])
    rs = out.get("reference_scenario")
    if rs:
        sm["reference_200x50_producer_MiB_per_s"] = rs["producer_MiB_per_s"]
        sm["reference_200x50_consumer_MiB_per_s"] = rs["consumer_MiB_per_s"]
        sm["reference_200x50_cpu_index_select_MiB_per_s"] = rs["cpu_index_select"]["MiB_per_s"]
        sm["reference_200x50_cpu_cores"] = rs["cpu_index_select"]["cores"]
    for note in ALLOC_NOTES:
        if note.get("what", "").startswith("qwen2_7b pool") and "seconds" in note:
            sm["headline_pool_alloc_s"] = note["seconds"]
            sm["headline_pool_alloc_fillers_GB"] = round(note["n_fillers"] * note["chunk_bytes"] / 1e9, 1)
            sm["headline_pool_chunks_other_half"] = f"{note['n_other_half']} of {note['n_chunks']}"
            break
    for k, v in sm.items():
        out["config"][k] = v
    out["summary"] = sm          # emitted last: the end of the line is what a truncated log keeps


if __name__ == "__main__":
    main()
