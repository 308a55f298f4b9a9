#!/usr/bin/env python3
"""Headline benchmark: SpMV GFLOP/s and fraction of the HBM roofline per matrix on one MI355X.

A "step" is one y = A x over the whole matrix with every array already resident in HBM: exactly the launches
the product call as_builder_spmv_device issues (the clear of y included where the graph needs it).  The
headline workload is BASELINE configuration 2: the 5-point Laplacian on a 2048 x 2048 grid (4,194,304 rows,
20,963,328 elements, fp32).  The operator graph and kernel are chosen by the search (tuning time is
reported, not timed as steps); the result is verified against the CPU CSR oracle before anything is timed.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C1..C5] [--tune-seconds S] [--pin GRAPH]

Without --workload the line carries C2 as the headline (value, roofline, cpu_baseline) and `per_matrix`: one
entry for each of the five BASELINE configurations (C1 plumbing case, C2 stencil, C3 power law, C4 FEM blocks,
C5 extreme irregularity), each with its GFLOP/s, roofline fraction (also on the CSR floor), whole-SpMV fraction,
tuning time, result check and CPU baseline.  C2, C5 and C1 are always searched; C3 and C4 are searched while the
wall-clock budget (--budget-seconds) allows and otherwise run the committed winners of earlier searches
(`tuning.mode` says which); a configuration that no longer fits the budget is recorded as skipped.
With --workload only that configuration is measured and it is the headline.  The roofline object is quoted on the
whole SpMV; with more than one row strip `roofline.dominant_kernel` holds the strip kernel that takes the longest,
timed alone, and "kernels" lists every strip kernel.  Two byte counts are given side by side: `algorithmic_bytes` /
`frac` count what the chosen format moves, the intermediate arrays its kernels write and read back included
(products, row sums: `scratch_bytes`, counted twice); `algorithmic_bytes_arrays_x_y` / `frac_arrays_x_y` count the
format arrays, x once and y once only (twice where y is cleared first).  `per_call_us` is one SpMV four ways: between
events on the stream (`kernels`, what `value` is made of), as a blocking product call, as an enqueue-only product
call, and as a replay of the allocation-free enqueue-only call captured into a HIP graph (null where the kernels'
scratch arrays do not fit the library's static array).

Prints ONE JSON line (rank 0).  One GPU only: --gpus above 1 exits with a message."""
import argparse
import gc
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "oracle"))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
T_START = time.perf_counter()

# name, generator, search budget (s) when measured alone / inside the five-matrix run, the committed winner of
# earlier searches as a --pin graph, rough seconds for generation + format build + checks (budget planning)
WORKLOADS = {
    "C1": ("C1: 4096x4096 uniform, 8 per row, fp32", "uniform_rows", {}, 45.0, 6.0, "|S1:m=512@512", 5.0),
    "C2": ("C2: 5-point Laplacian, 2048x2048 grid, 4194304 rows, fp32", "laplacian_5pt", {"grid": 2048}, 45.0, 30.0,
           "S5,256,1,dia", 12.0),
    "C3": ("C3: power-law row lengths (Zipf 1.8, mean 16, max 200000), 2000000 rows, uniform columns, fp32", "power_law",
           {}, 90.0, 60.0, "sort+div48|T1@1024|T2:slice=16384,group=4096@1024", 30.0),
    "C4": ("C4: FEM-like dense 3x3 blocks, 27 block columns per block row in a +-2000 band, 1000002 rows, fp64",
           "fem_blocks", {}, 45.0, 25.0, "|T1:slice=16384,group=4092@1024,runs,own,blk3", 35.0),
    "C5": ("C5: 8000000 rows of 1-3 elements + 800 rows of 50000-1000000 elements, uniform columns, fp64",
           "extreme_irregular", {"target_nnz": 60_000_000}, 150.0, 75.0,
           "sort+div16|T1:slice=16384,group=4096@1024|T2:slice=16384,group=4096@1024", 45.0),
}
# the rocprofv3 summary that covers each configuration's kernels
PROFILE_OF = {"C2": "profiles/spmv_ell_c2_laplacian_hbm_traffic.txt", "C3": "profiles/spmv_tile_product_bin_c3_power_law.txt",
              "C4": "profiles/spmv_tile_c4_fem_blocks.txt", "C5": "profiles/spmv_tile_product_bin_c5_extreme_irregular.txt"}
# HBM bytes per launch, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs, each scaled by what the same
# counter reads for the plain copy kernel of --copy-calibration), by the first 16 hex digits of the SHA-256 of the
# generated module source: a graph whose kernels changed in any way since it was profiled reports null and names the
# profile instead.  The figures live beside the summaries they come from.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic_by_graph_hash.json")


def measured_traffic(graph_hash):
    try:
        with open(TRAFFIC_FILE) as f:
            entry = json.load(f).get(graph_hash)
    except (OSError, ValueError):
        return None
    return entry["bytes"] if entry else None


def cpu_baseline(rows, r, c, v, x, nnz, seconds):
    """The CPU CSR SpMV oracle (own restatement of the merge-path OpenMP baseline) on this host's cores."""
    import numpy as np
    import spmv_oracle as O
    threads = min(O.max_threads(), os.cpu_count() or 1)
    rp = O.coo_to_csr(rows, r)
    ci = c.astype(np.uint32)
    for _ in range(3):
        O.spmv_csr_merge(rp, ci, v, x, threads=threads)
    times = []
    t_end = time.perf_counter() + seconds
    while len(times) < 10 or (time.perf_counter() < t_end and len(times) < 200):
        t0 = time.perf_counter()
        O.spmv_csr_merge(rp, ci, v, x, threads=threads)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {"value": round(2.0 * nnz / med / 1e9, 3), "unit": "GFLOP/s", "cores": threads, "kind": "port",
            "sample": "same matrix and x, OpenMP merge-path CSR, median of %d runs after 3 warm-ups" % len(times)}


class _Pinned:
    report, dense_strategy, n_sub, seconds_to_best, candidates, failed_candidates = "", 1, 1, 0.0, 0, 0


def build_pinned(m, pin):
    """A fixed graph instead of the search: 'S5,128,1[,rel|dia]' (one strip: skeleton, threads, rows per lane) or
    'sort+div16|T1@1024|S1:m=128@128' (dense operators | one skeleton per strip, kernels one after the other)."""
    import alphasparse_amd as A
    from alphasparse_amd import _capi as K, skeletons as SK
    res = _Pinned()
    if "|" not in pin:
        skel, threads, vec, *more = pin.split(",")
        m.execute_strategy(K.COMPRESS_NONE)
        templates = SK.apply_skeleton(m, 0, skel)
        b = A.Builder(m)
        b.set_template(0, templates[0])
        if "rel" in more and not b.set_relative_columns(0):
            raise SystemExit("bench.py: relative columns do not apply to this graph")
        if "dia" in more and not b.set_diagonal_columns(0):
            raise SystemExit("bench.py: diagonal columns do not apply to this graph")
        b.set_launch(0, thread_num_in_block=int(threads), vec_width=int(vec))
        return b, res
    dense, *strips = pin.split("|")
    serial = True
    for op in filter(None, dense.split("+")):
        if op == "sort":
            m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
            res.dense_strategy = 3
        elif op == "par":
            serial = False        # the strip kernels on concurrent streams instead of one after the other
        elif op.startswith("div"):
            low = int(op[3:])
            m.execute_strategy(K.DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, -1, (low, low, 2, 0))
            res.dense_strategy = max(res.dense_strategy, 2)
        else:
            raise SystemExit("bench.py: unknown dense operator %r in --pin" % op)
    m.execute_strategy(K.COMPRESS_NONE)
    res.n_sub = m.info()["n_sub"]
    if len(strips) != res.n_sub:
        raise SystemExit("bench.py: --pin names %d strips, the matrix has %d" % (len(strips), res.n_sub))
    chosen = []
    for s, spec in enumerate(strips):
        spec, _, launch = spec.partition("@")
        skel, _, kw = spec.partition(":")
        kw = {k: int(x) for k, x in (p.split("=") for p in filter(None, kw.split(",")))}
        words = [x for x in launch.split(",") if x]
        blocks = [int(x[3:]) for x in words if x.startswith("blk")]
        chosen.append((SK.apply_skeleton(m, s, skel, **kw)[0], [int(x) for x in words if x.isdigit()], "runs" in words, "own" in words,
                       blocks[0] if blocks else 0))
    b = A.Builder(m)
    for s, (tp, launch, runs, own, blocks) in enumerate(chosen):
        b.set_template(s, tp)
        if runs and not b.set_column_runs(s):
            raise SystemExit("bench.py: the column-run form does not apply to strip %d" % s)
        if own and not b.set_row_ownership(s):
            raise SystemExit("bench.py: row ownership does not apply to strip %d" % s)
        if blocks and not b.set_row_blocks(s, blocks):
            raise SystemExit("bench.py: the rows of strip %d do not come in blocks of %d" % (s, blocks))
        if launch:
            b.set_launch(s, thread_num_in_block=launch[0], vec_width=launch[1] if len(launch) > 1 else 0)
    b.set_serial_launch(serial)
    return b, res


def measure(key, steps, warmup, tune_seconds, pin, cpu_seconds, copy_calibration=False, echo_report=False):
    """One configuration end to end: generate, search (or pinned graph), check against the oracle, time.
    Returns the full result object of that configuration."""
    import numpy as np
    import alphasparse_amd as A
    from alphasparse_amd import _capi as K, synthetic as S
    import spmv_oracle as O

    name, gen, gen_kw, _, _, _, _ = WORKLOADS[key]
    t_gen = time.perf_counter()
    rows, cols, r, c, v, x = getattr(S, gen)(**gen_kw)
    nnz = len(r)
    val_dtype = K.DOUBLE if v.dtype == np.float64 else K.FLOAT
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), val_dtype, wave=64)
    gen_s = time.perf_counter() - t_gen

    t0 = time.perf_counter()
    if pin:
        b, res = build_pinned(m, pin)
    else:
        res = A.find_best_graph(m, total_time_s=tune_seconds, device=0)
        b = res.build_best()
    tune_s = time.perf_counter() - t0
    b.compile().upload(0)
    if echo_report and res.report:
        print(res.report, file=sys.stderr)   # the best operator graph, as the search reports it

    # correctness gate before any timing
    y = b.spmv(x)
    y_ref, mag = O.spmv_csr(O.coo_to_csr(rows, r), c.astype(np.uint32), v, x)
    rel, ratio, tol = O.check_y(y, y_ref, mag, v.dtype.type)
    if not (rel <= tol and ratio <= 1.0):
        raise RuntimeError("%s: result check failed (rel L2 %.3e, per-row ratio %.2f)" % (key, rel, ratio))
    del y, y_ref, mag

    L = K.lib()
    copy_gbs = None
    if copy_calibration:
        import ctypes as C
        L.as_selftest_copy.argtypes = [C.c_int, C.c_uint64, C.c_int, C.POINTER(C.c_float)]
        ms = C.c_float(0)
        K.check(L.as_selftest_copy(0, 256 << 20, 20, C.byref(ms)), L)
        copy_gbs = 2.0 * (256 << 20) / (ms.value * 1e-3) / 1e9
    b.set_x(x)
    b.time(max(1, warmup))                 # W untimed steps
    L.as_hip_device_sync()
    t0 = time.perf_counter()
    kernel_ms, _ = b.time(steps)           # exactly K steps, events on the launch stream inside
    L.as_hip_device_sync()
    wall = time.perf_counter() - t0
    gflops = 2.0 * nnz * steps / wall / 1e9
    bytes_per_step = b.algorithmic_bytes()
    per_launch_s = kernel_ms * 1e-3 / steps
    achieved = bytes_per_step / per_launch_s / 1e9
    # every strip kernel alone (events on its launch stream): algorithmic bytes = its format arrays + x once +
    # the y rows of its strip (twice when it accumulates atomically into the cleared y)
    vs = v.dtype.itemsize
    reps = max(50, steps // 4)
    kernels = []
    for s in range(int(res.n_sub)):
        ms, fmt_bytes, strip_rows, atom = b.time_sub_matrix(s, reps)
        us = ms * 1e3 / reps
        kb = fmt_bytes + cols * vs + strip_rows * vs * (2 if atom else 1)
        kernels.append({"sub_matrix": s, "kernel_us": round(us, 3), "algorithmic_bytes": kb,
                        "scratch_bytes": b.scratch_bytes(s), "algorithmic_bytes_arrays_x_y": kb - 2 * b.scratch_bytes(s),
                        "achieved_gbs": round(kb / us / 1e3, 1), "frac": round(kb / us / 1e3 / HBM_PEAK_GBS, 4),
                        "frac_arrays_x_y": round((kb - 2 * b.scratch_bytes(s)) / us / 1e3 / HBM_PEAK_GBS, 4),
                        "strip_rows": strip_rows})
        try:  # templates with two kernels: each launched alone
            kernels[-1]["pass_us"] = [round(b.time_sub_matrix_pass(s, which, reps) * 1e3 / reps, 3) for which in (1, 2)]
        except A.AlphaSparseError:
            pass
    dominant = max(kernels, key=lambda k: k["kernel_us"])
    roof_us, roof_bytes = per_launch_s * 1e6, bytes_per_step
    csr_floor = nnz * (v.dtype.itemsize + 4) + (rows + 1) * 4 + (rows + cols) * v.dtype.itemsize
    sync_ok, sync_ms, sync_gf = A.part_execute_code_builder(b, [], 200)
    # the product calls on device buffers of the caller, wall clock per call: the blocking call (a wait per SpMV)
    # and the enqueue-only call (N calls, one wait)
    dx, dy = A.DeviceArray(x), A.DeviceArray(np.zeros(rows, v.dtype))
    calls = 300
    for _ in range(20):
        b.spmv_device_async(dx, dy, None)
    b.sync()
    t0 = time.perf_counter()
    for _ in range(calls):
        b.spmv_device_async(dx, dy, None)
        b.sync()
    per_call_sync_us = (time.perf_counter() - t0) / calls * 1e6
    t0 = time.perf_counter()
    for _ in range(calls):
        b.spmv_device_async(dx, dy, None)
    b.sync()
    per_call_async_us = (time.perf_counter() - t0) / calls * 1e6
    # ... and the allocation-free enqueue-only call recorded once by a stream capture and replayed as a HIP graph
    # (null where the kernels' scratch arrays do not fit the library's static array)
    per_call_graph_us = None
    try:
        if 0 <= b.static_scratch_need() <= (64 << 20):
            stream = A.Stream()
            b.spmv_device_async(dx, dy, stream, no_alloc=True)
            stream.sync()
            stream.capture_begin()
            b.spmv_device_async(dx, dy, stream, no_alloc=True)
            graph = stream.capture_end()
            for _ in range(20):
                stream.graph_launch(graph)
            stream.sync()
            t0 = time.perf_counter()
            for _ in range(calls):
                stream.graph_launch(graph)
            stream.sync()
            per_call_graph_us = (time.perf_counter() - t0) / calls * 1e6
            y_graph = dy.get()
            rel_g, ratio_g, tol_g = O.check_y(y_graph, *O.spmv_csr(O.coo_to_csr(rows, r), c.astype(np.uint32), v, x), v.dtype.type)
            if not (rel_g <= tol_g and ratio_g <= 1.0):
                raise RuntimeError("%s: the replayed graph's y differs (rel L2 %.3e)" % (key, rel_g))
            stream.graph_destroy(graph)
            stream.destroy()
    except A.AlphaSparseError as e:
        print("[bench] %s: graph replay not timed: %s" % (key, str(e)[:200]), file=sys.stderr)
        per_call_graph_us = None
    dx.free()
    dy.free()
    scratch = b.scratch_bytes()
    bytes_arrays_x_y = bytes_per_step - 2 * scratch

    templates = [b.describe(s)["template"] for s in range(int(res.n_sub))]
    launches = [b.get_launch(s) for s in range(int(res.n_sub))]
    source = b.kernel_source()
    graph_hash = hashlib.sha256(source.encode()).hexdigest()[:16]

    def column_form(sub):  # how the template of this sub-matrix stores its columns
        d = b.describe(sub)
        if any(k.startswith("diagonal_offset_") for k in d):
            return "diagonal (computed, no array)"
        if "col_run_mask" in d["arrays"]:
            return "runs of consecutive columns"
        if d["template"] == "DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS" and d["arrays"]["col_index_arr"][0] == "UNSIGNED_SHORT" \
                and "(short)" in source:
            return "16-bit relative"
        return "explicit"
    whole_gbs = bytes_per_step / per_launch_s / 1e9
    out = {
        "metric": "SpMV GFLOP/s and % of HBM BW roofline per matrix, 1xMI355X",
        "value": round(gflops, 2), "unit": "GFLOP/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(wall * 1e3 / steps, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f64" if v.dtype == np.float64 else "f32", "data": "synthetic",
        "config": {"workload": name, "rows": rows, "nnz": nnz, "pinned": pin,
                   "dense_strategy": int(res.dense_strategy), "sub_matrices": int(res.n_sub),
                   "template": templates, "launch": launches,
                   "columns": [column_form(s) for s in range(int(res.n_sub))],
                   "rows_owned": ["run_row_group" in b.describe(s)["arrays"] for s in range(int(res.n_sub))],
                   "row_block": [int(b.describe(s).get("row_block", 1)) for s in range(int(res.n_sub))],
                   "clears_y": b.clears_y(), "graph_hash": graph_hash},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic(graph_hash), "traffic_profile": PROFILE_OF.get(key),
                     "kernel_us": round(roof_us, 3), "algorithmic_bytes": roof_bytes,
                     "scratch_bytes": scratch, "algorithmic_bytes_arrays_x_y": bytes_arrays_x_y,
                     "frac_arrays_x_y": round(bytes_arrays_x_y / per_launch_s / 1e9 / HBM_PEAK_GBS, 4),
                     "kernel": "whole SpMV: " + " + ".join("spmv_%d (%s)" % (s_, templates[s_]) for s_ in range(int(res.n_sub))),
                     "dominant_kernel": {"kernel": "spmv_%d (%s)" % (dominant["sub_matrix"], templates[dominant["sub_matrix"]]),
                                         "kernel_us": dominant["kernel_us"], "algorithmic_bytes": dominant["algorithmic_bytes"],
                                         "achieved": dominant["achieved_gbs"], "frac": dominant["frac"],
                                         "frac_arrays_x_y": dominant["frac_arrays_x_y"]},
                     "csr_floor_bytes": csr_floor,
                     "csr_floor_frac": round(csr_floor / per_launch_s / 1e9 / HBM_PEAK_GBS, 4)},
        "whole_spmv": {"us": round(per_launch_s * 1e6, 3), "algorithmic_bytes": bytes_per_step,
                       "achieved_gbs": round(whole_gbs, 1), "frac": round(whole_gbs / HBM_PEAK_GBS, 4),
                       "algorithmic_bytes_arrays_x_y": bytes_arrays_x_y,
                       "frac_arrays_x_y": round(bytes_arrays_x_y / per_launch_s / 1e9 / HBM_PEAK_GBS, 4),
                       "kernel_gflops": round(2.0 * nnz / per_launch_s / 1e9, 2)},
        "per_call_us": {"kernels": round(per_launch_s * 1e6, 3), "blocking_call": round(per_call_sync_us, 3),
                        "enqueue_only_call": round(per_call_async_us, 3),
                        "graph_replay": None if per_call_graph_us is None else round(per_call_graph_us, 3), "calls": calls},
        "kernels": kernels,
        "tuning": {"mode": "pinned" if pin else "search", "seconds": round(tune_s, 2),
                   "seconds_to_best": round(res.seconds_to_best, 2),
                   "candidates": int(res.candidates), "failed": int(res.failed_candidates),
                   "generation_seconds": round(gen_s, 2)},
        "per_launch_sync_gflops": round(sync_gf, 2) if sync_ok else None,
        "check": {"rel_l2": float("%.3e" % rel), "per_row_bound_ratio": round(ratio, 4)},
    }
    if copy_gbs is not None:
        out["copy_kernel_gbs"] = round(copy_gbs, 1)
    b.close()
    del b, res, m
    if cpu_seconds > 0:
        out["cpu_baseline"] = cpu_baseline(rows, r, c, v, x, nnz, cpu_seconds)
    del r, c, v, x
    gc.collect()
    return out


def per_matrix_entry(key, full):
    """The part of a configuration's result that the per_matrix list carries."""
    e = {"workload": key, "gflops": full["value"], "ms_per_step": full["ms_per_step"], "steps": full["steps"],
         "dtype": full["dtype"], "rows": full["config"]["rows"], "nnz": full["config"]["nnz"],
         "graph": {k: full["config"][k] for k in ("dense_strategy", "sub_matrices", "template", "launch", "columns",
                                                   "rows_owned", "row_block", "clears_y", "graph_hash", "pinned")},
         "roofline": {k: full["roofline"][k] for k in ("frac", "achieved", "kernel", "kernel_us", "algorithmic_bytes",
                                                       "scratch_bytes", "algorithmic_bytes_arrays_x_y", "frac_arrays_x_y",
                                                       "dominant_kernel", "csr_floor_bytes", "csr_floor_frac", "traffic",
                                                       "traffic_profile")},
         "whole_spmv": full["whole_spmv"], "per_call_us": full["per_call_us"], "kernels": full["kernels"],
         "tuning": full["tuning"], "check": full["check"]}
    if "cpu_baseline" in full:
        e["cpu_baseline"] = full["cpu_baseline"]
    return e


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--tune-seconds", type=float, default=None,
                    help="search budget; with --workload the default is 45 s (C1, C2, C4), 90 s (C3), 150 s (C5); in the "
                         "five-matrix run 6 / 30 / 60 / 25 / 75 s for C1..C5")
    ap.add_argument("--workload", default=None, choices=["C1", "C2", "C3", "C4", "C5"],
                    help="measure this configuration only (default: all five, C2 as the headline)")
    ap.add_argument("--budget-seconds", type=float, default=420.0,
                    help="five-matrix run: wall-clock budget of the whole program; C3 / C4 fall back to their committed "
                         "winners and a configuration is skipped when the budget would be exceeded")
    ap.add_argument("--pin", default=None, metavar="SKELETON,THREADS,VEC | DENSE|STRIP0|STRIP1...",
                    help="with --workload: skip the search and run a fixed graph: S5,128,1 (ELL, 128 threads, 1 row per lane; S5,128,1,rel with 16-bit relative columns), or with "
                         "row strips 'sort+div16|T1@1024|S1:m=128@128' = coarse sort, two strips at row length 16 ('+par': strip kernels on concurrent streams), strip 0 "
                         "skeleton T1 with 1024 threads, strip 1 skeleton S1 (m = 128) with 128 threads, kernels one after "
                         "the other ('@1024,runs': the tile template in its column-run form, '@1024,own': under row ownership); used for profiling runs that must all "
                         "measure the same kernels")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch a plain 256 MiB copy kernel (as_copy_words) 20 times: reference traffic for "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (rows would shard across GPUs with x "
              "replicated and no reduction).  Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if args.pin and not args.workload:
        print("bench.py: --pin needs --workload", file=sys.stderr)
        sys.exit(2)

    import alphasparse_amd as A
    if A.device_count() < 1:
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)

    if args.workload:
        tune = args.tune_seconds if args.tune_seconds is not None else WORKLOADS[args.workload][3]
        try:
            out = measure(args.workload, args.steps, args.warmup, tune, args.pin, 0 if args.no_cpu_baseline else 15.0,
                          args.copy_calibration, echo_report=True)
        except RuntimeError as e:
            print("bench.py: %s" % e, file=sys.stderr)
            sys.exit(1)
        print(json.dumps(out))
        return

    # ---- all five configurations: C2 first (the headline), then the one whose search the configuration demands ----
    results = {}
    pm_steps = max(args.steps, 200)   # the other matrices: enough launches for a steady rate
    for key in ("C2", "C5", "C3", "C4", "C1"):
        _, _, _, _, tune_all, pinned, fixed_s = WORKLOADS[key]
        tune = args.tune_seconds if args.tune_seconds is not None else tune_all
        cpu_s = 0 if args.no_cpu_baseline else (15.0 if key == "C2" else 5.0)
        left = args.budget_seconds - (time.perf_counter() - T_START)
        pin = None
        if key in ("C3", "C4") and left < fixed_s + tune + cpu_s + 15.0:
            pin = pinned          # no room for a search: the committed winner
        if key != "C2" and left < fixed_s + cpu_s + (0 if pin else tune):
            results[key] = {"workload": key, "skipped": "budget",
                            "seconds_left": round(left, 1)}
            continue
        print("[bench] %s: %s, %.0f s of budget left" % (key, "pinned graph" if pin else "search %.0f s" % tune, left),
              file=sys.stderr, flush=True)
        try:
            full = measure(key, args.steps if key == "C2" else pm_steps, args.warmup, tune, pin, cpu_s,
                           echo_report=(key == "C2"))
        except RuntimeError as e:
            if key == "C2":
                print("bench.py: %s" % e, file=sys.stderr)
                sys.exit(1)
            results[key] = {"workload": key, "failed": str(e)}
            continue
        results[key] = full
    out = dict(results["C2"])
    out["per_matrix"] = [per_matrix_entry(k, results[k]) if "value" in results[k] else results[k]
                         for k in ("C1", "C2", "C3", "C4", "C5")]
    out["wall_seconds"] = round(time.perf_counter() - T_START, 1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
