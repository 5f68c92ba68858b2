"""bench.py's contract with whatever runs it, checked without a GPU: more than one GPU is refused with a
message, the summary block carries every part of a default run under `config` and as the last key of the
line, and the HBM traffic ratios the line replays belong to the kernel sources as they are now."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0 and "one GPU" in r.stderr and not r.stdout.strip()


def test_traffic_ratios_belong_to_the_kernels_as_they_are():
    """`roofline.traffic` multiplies a run's algorithmic bytes by a ratio read from rocprofv3 counters earlier;
    the line reports it only while the kernel source is the one the counters were read from."""
    import bench
    for fname, digest in bench.TRAFFIC_MEASURED_AT.items():
        assert bench.kernel_source_digest(fname) == digest, (
            f"{fname} changed since its FETCH_SIZE / WRITE_SIZE counters were read: re-measure (profiles/) and update "
            "MEASURED_TRAFFIC_RATIO and TRAFFIC_MEASURED_AT in bench.py")
    ratio, src = bench.traffic_ratio("qwen2_7b", "gather")
    assert 0.9 < ratio < 1.1 and "profiles/" in src
    assert bench.traffic_ratio("no_such_workload", "gather") == (None, None)


def test_summary_block_is_flat_complete_and_last():
    import bench
    k = lambda g: {"GBps": g, "avg_ms": 1.0, "alg_bytes": 1}
    cfg = lambda v, s=True: {"value": v, "gather": dict(k(v), frac=v / 8000), "scatter": dict(k(v), frac=v / 8000) if s else None}
    fp = {f"{d}_{m}": {"GBps": 50.0} for d in ("gather", "scatter") for m in ("auto", "pipelined_kernel", "pipelined")}
    fp["what"] = "text"
    out = {"value": 6500.0, "config": {"workload": "w"}, "kernels": {"gather": k(6400.0), "scatter": k(6600.0)},
           "other_layout": {"value": 6400.0}, "torch_alloc": {"value": 6300.0, "kernels": {"gather": k(6200.0), "scatter": k(6400.0)}},
           "configs": {"qwen2_1p5b": cfg(6300.0, False), "llama3_70b_fp8": cfg(6350.0)},
           "staging": {"host_link_GBps": 55.7, "plain_d2h_GBps": {"median": 57.1}, "plain_h2d_GBps": {"median": 57.6},
                       "frac_of_plain_d2h": 0.97, "scatter_frac_of_plain_h2d": 0.96,
                       "min_frac_over_cells": {"gather_to_host": 0.95, "scatter_from_host": 0.92},
                       "median_frac_over_cells": {"gather_to_host": 0.98, "scatter_from_host": 0.96},
                       "first_pass": fp, "wait_for_full_rate_copies": {"seconds": 0.5}},
           "layout_change": {"value": 6200.0, "kernels": {"load": k(6500.0), "store": k(6000.0)}},
           "reference_scenario": {"producer_MiB_per_s": 2.5e6, "consumer_MiB_per_s": 3e7,
                                  "cpu_index_select": {"MiB_per_s": 8e4, "cores": 16}}}
    bench.add_summary(out)
    sm = out["summary"]
    for key in ("headline_gather_frac", "torch_alloc_value_GBps", "qwen2_1p5b_gather_frac", "llama3_70b_fp8_scatter_frac",
                "staging_auto_gather_frac_median", "staging_gather_frac_min_over_cells", "staging_first_pass_gather_auto_GBps",
                "staging_first_pass_scatter_pipelined_GBps", "layout_change_store_frac", "reference_200x50_producer_MiB_per_s",
                "reference_200x50_cpu_cores"):
        assert key in sm and out["config"][key] == sm[key], key
    assert "qwen2_1p5b_scatter_frac" not in sm                        # that configuration only gathers
    assert all(not isinstance(v, (dict, list)) for v in sm.values())  # flat: a record that keeps scalars keeps it all
    assert sm["headline_gather_frac"] == 0.8
    # emitted as the last key of the line
    import io
    import contextlib
    buf = io.StringIO()
    with contextlib.redirect_stdout(buf):
        bench.emit(out)
    assert list(json.loads(buf.getvalue()).keys())[-1] == "summary"


def test_live_traffic_is_computed_from_the_two_counters_and_their_calibration(tmp_path):
    """The figures `roofline.traffic` is made of when the run measures them itself: per-dispatch means of each
    counter for the dominant kernel, each scaled by the same counter's reading for the plain 2 GiB copy. The
    counter files here are written by hand in rocprofv3's column layout: FETCH_SIZE counting half the KiB a
    kernel fetches (as on MI355X), WRITE_SIZE all of them, two instances per dispatch, other kernels in between."""
    import bench
    head = '"Correlation_Id","Dispatch_Id","Kernel_Name","Counter_Name","Counter_Value"\n'
    kib = (2 << 30) // 1024
    alg = 2 * 3 * (1 << 30)                                            # the kernel reads 3 GiB and writes 3 GiB
    def rows(counter, copy_val, dom_val):
        out, did = [], 0
        for name, val, n in (("void bikv::copy_runs_wave_kernel<true, true, 64, true>(bikv::RunArgs)", copy_val, 3),
                             ("void at::native::vectorized_elementwise_kernel<4>(int)", 12345.0, 2),
                             ("void bikv::tile_move_wave_kernel<0, 2, 64>(bikv::MoveArgs)", dom_val, 4),
                             ("void bikv::tile_move_wave_kernel<1, 2, 64>(bikv::MoveArgs)", 7.0, 4)):
            for _ in range(n):
                did += 1
                for inst in range(2):                                   # two rows of one dispatch add up
                    out.append(f'{did},{did},"{name}","{counter}",{val / 2}\n')
                out.append(f'{did},{did},"{name}","SOME_OTHER_COUNTER",1.0\n')
        return head + "".join(out)
    f, w = tmp_path / "f.csv", tmp_path / "w.csv"
    f.write_text(rows("FETCH_SIZE", kib / 2, 3 * (1 << 20) / 2 * 1.01))   # 1 % more fetched than the algorithm needs
    w.write_text(rows("WRITE_SIZE", kib, 3 * (1 << 20)))
    fm = bench.counter_means(str(f), "FETCH_SIZE", "tile_move_wave_kernel<0")
    wm = bench.counter_means(str(w), "WRITE_SIZE", "tile_move_wave_kernel<0")
    assert fm["copy"][0] == 3 and fm["dominant"][0] == 4 and abs(fm["copy"][1] - kib / 2) < 1e-6
    live, note = bench.traffic_from_counters(fm, wm, alg)
    assert abs(note["fetch_scale_from_plain_copy"] - 2.0) < 1e-9 and abs(note["write_scale_from_plain_copy"] - 1.0) < 1e-9
    assert note["written_bytes"] == 3 << 30 and abs(note["fetched_bytes"] - 1.01 * (3 << 30)) < 2
    assert live == note["fetched_bytes"] + note["written_bytes"] and note["ratio_to_algorithmic"] == 1.005
    # counters that make no sense against the calibration are not reported
    bad, note = bench.traffic_from_counters({"copy": (3, kib * 100.0), "dominant": fm["dominant"]}, wm, alg)
    assert bad is None and "skipped" in note
