#!/usr/bin/env python3
"""Benchmark of the fused merge-path SpMV / map + reducer + aggregator path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--size N] [--all]

A step is one ``merged_spmv_launch`` of the workload's fused sub-graph (all kernels of the launch,
inputs resident in HBM).  The headline workload is the 3-D 7-point Poisson operator on a 256^3 grid in
float64: fused ``y = A x`` and ``x . y``; the other four workloads (R-MAT scale 22 in float32 - the second
target workload -, shallow water, spring-mass, 2-D Laplacian) are timed in the same run and reported under
``other_workloads`` with their own roofline and CPU baseline.  One JSON line is printed:

* ``value``         effective GB/s = algorithmic bytes per step / (wall time of exactly K steps / K)
                    (every streamed array once, every gathered source once, every output once)
* ``step_ms_*``     the same steps one by one, each bracketed by HIP events on the launch stream:
                    median and minimum over the K launches
* ``roofline``      the dominant kernel alone: algorithmic bytes / its mean duration over K launches,
                    measured with HIP events around that kernel on the launch stream, against the
                    8 TB/s HBM peak (median and minimum are reported beside the mean)
* ``cpu_baseline``  the CPU oracle (a port of the reference's OpenMP path) on the same inputs, timed on
                    this host's cores, and the parity of the GPU result against it (row by row,
                    relative to max(|reference|, sum of |contributions| of the row))

The exit code is 1 and ``value`` is null when the GPU result is outside the tolerance.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
DEFAULT_SIZE = {"poisson3d": 256, "rmat": 22, "spring_mass": 100, "shallow_water": 1_000_000, "laplacian2d": 256}
DTYPE_TAG = {"float32": "f32", "float64": "f64", "int64": "i64"}
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic.md")
WORKLOAD_NOTES = {
    "spring_mass": "rest length = lattice spacing h (the jitter is the displacement); with rest length = initial "
                   "length every force and the energy would be exactly zero",
    "shallow_water": "cells renumbered along a Morton curve through their centroids before the half-edges are "
                     "sorted by destination cell (the triangulation's own numbering has no locality)",
    "laplacian2d": "the reference's CPU-sized case: 3.4 MB of algorithmic bytes are 0.4 us at the HBM peak, so the step is "
                   "the latency of its two kernel launches and the roofline fraction says nothing about the kernel",
}


def host_threads() -> int:
    n = int(os.environ.get("OMP_NUM_THREADS", "0") or 0)
    if n <= 0:
        n = os.cpu_count() or 1
    return max(1, min(n, 256))          # 256 = size of the reference's per-thread carry arrays


def measured_traffic(workload_name: str, kernel: str, policy: str):
    """HBM bytes per launch of ``kernel`` on ``workload_name`` from the table in profiles/hbm_traffic.md
    (rocprofv3 FETCH_SIZE / WRITE_SIZE per dispatch, scaled by the copy-kernel calibration quoted there), or
    None when the table has no row for this kernel, workload and policy."""
    try:
        with open(TRAFFIC_TABLE) as f:
            text = f.read()
    except OSError:
        return None
    for line in text.splitlines():
        cells = [c.strip().strip("`") for c in line.strip().strip("|").split("|")]
        if len(cells) >= 7 and cells[0] == workload_name and cells[1] == kernel and cells[2] == policy:
            try:
                fetch_kib, write_kib, f_fetch, f_write = (float(re.sub(r"[ ,]", "", c)) for c in cells[3:7])
            except ValueError:
                return None
            return {"bytes": int((fetch_kib * f_fetch + write_kib * f_write) * 1024),
                    "source": "profiles/hbm_traffic.md"}
    return None


def machine_mix_rate(ext, w, dtype_name, write_bytes, launches=30):
    """What the memory system delivers for this workload's mix of reads and writes without any arithmetic:
    the calibration kernel (flexspmv_amd/csrc/flex_calibrate.hip) with one block per tile of the launch, each
    reading and writing its share of the algorithmic bytes (reads rounded up to 4 KB per tile, writes to 8
    bytes), tiles dealt to the XCDs as the launch deals them.  Returns a dict for the bench line, or None
    for sub-graphs without tiles of this kind or when the calibration library is not built."""
    import ctypes

    import torch

    from flexspmv_amd import build as fbuild
    from flexspmv_amd.binding import DTYPE_CODES
    if not ext.signature["has_reducer"] or not os.path.exists(fbuild.CALIBRATE_LIBRARY):
        return None
    lib = ctypes.CDLL(fbuild.CALIBRATE_LIBRARY)
    fn = lib.flexspmv_calibrate_stream_mix
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
                   ctypes.c_int32, ctypes.c_void_p]
    fn.restype = ctypes.c_int
    tl = (ctypes.c_int32 * 6)()
    if ext._lib.flexspmv_tiling(DTYPE_CODES[dtype_name], w.num_rows, w.ne, tl) != 0:
        return None
    tiles, snapped = int(tl[0]), int(tl[2]) > 0
    read_per_tile = -(-(w.algorithmic_bytes - write_bytes) // tiles // 4096) * 4096
    write_per_tile = min(2048, -(-write_bytes // tiles // 8) * 8)
    src = torch.ones(tiles * read_per_tile, dtype=torch.uint8, device="cuda:0")
    dst = torch.empty(tiles * max(write_per_tile, 8), dtype=torch.uint8, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream

    def run(write, count):
        """Mean time of `count` launches issued back to back, after 10 untimed ones."""
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(10 + count):
            if i == 10:
                e0.record()
            rc = fn(src.data_ptr(), dst.data_ptr(), tiles, read_per_tile, write, 4 if snapped else 0, 0, stream)
            if rc != 0:
                raise RuntimeError(f"calibration kernel failed ({rc})")
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) / count

    for _ in range(2):       # the first series also serves as warm-up of the second
        ms_mix = run(write_per_tile, launches)
        ms_read = run(0, launches)
    moved = tiles * (read_per_tile + write_per_tile)
    return {"kernel": "one block per tile: 16-byte loads of the tile's share of the reads, 8-byte stores of its "
                      "share of the writes, no arithmetic (flexspmv_amd/csrc/flex_calibrate.hip)",
            "tiles": tiles, "read_bytes": tiles * read_per_tile, "write_bytes": tiles * write_per_tile,
            "ms": ms_mix, "gbs": moved / ms_mix / 1e6,
            "reads_only_ms": ms_read, "reads_only_gbs": tiles * read_per_tile / ms_read / 1e6}


def time_workload(w, steps, warmup, library=None, calibrate=False, compare_sources=True):
    """GPU leg: returns (result dict, outputs of the last launch as numpy arrays)."""
    import torch

    from flexspmv_amd import workloads as W
    from flexspmv_amd.binding import HipExtension, load_named

    ext = HipExtension(library, allow_variant=True) if library else load_named(w.graph, build_if_missing=False)
    args = W.launch_arguments(w, ext.param_names(), "cuda:0")
    # Untimed warm-up: W launches, and in any case launches for 60 ms.  Building a workload keeps the host
    # busy for seconds while the GPU idles and clocks down; a handful of sub-millisecond launches is not
    # enough to bring the clocks back up, and a burst of work that follows an idle stretch - a few
    # milliseconds are enough - goes through a transient first (rocprofv3's per-dispatch durations of the
    # Poisson kernel: 307 us for the first 6 launches, 315 - 328 for the next 30, back to 303 - 307 after 17 ms).
    # Every timed series below therefore starts with the same warm-up.  The pause before it lets the worker threads of the host-side
    # generators (numpy / torch CPU kernels), which spin for a while after their last parallel region,
    # get out of the launch thread's way.
    def warm_up():
        out = None
        t0 = time.perf_counter()
        done = 0
        while done < max(warmup, 1) or time.perf_counter() - t0 < 0.06:
            out = ext.merged_spmv_launch(*args)
            done += 1
            if done % 16 == 0:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        return out

    time.sleep(0.3)
    outs = warm_up()

    # the timed region: exactly K launches between two synchronisations
    t0 = time.perf_counter()
    for _ in range(steps):
        outs = ext.merged_spmv_launch(*args)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps

    # A region of K launches of a small workload is over in a millisecond and one hiccup of the host doubles
    # it: such a workload gets six more regions of K launches each, and the median of the seven is reported
    # beside the first.
    region_ms = [ms_per_step]
    if ms_per_step * steps < 10.0:
        for _ in range(6):
            t0 = time.perf_counter()
            for _ in range(steps):
                ext.merged_spmv_launch(*args)
            torch.cuda.synchronize()
            region_ms.append((time.perf_counter() - t0) * 1e3 / steps)
    region_ms.sort()

    # the same launches one by one, each between two events on the launch stream
    step_ms = []
    for _ in range(steps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        ext.merged_spmv_launch(*args)
        e1.record()
        e1.synchronize()
        step_ms.append(e0.elapsed_time(e1))
    step_ms.sort()

    # Launches find the tile table of the launch before in their scratch and confirm it, block by block,
    # against the row pointer they are given (flexspmv.h: the tile table); the timed region above follows the
    # warm-up on the same matrix, so its blocks confirm and no search runs.  Beside it: the same K launches
    # with every boundary searched afresh on every launch, as the reference does (a search kernel in front of
    # large launches) ...
    ms_per_step_search = None
    from flexspmv_amd.binding import FLAG_SEARCH_TILES
    if ext.signature["has_reducer"] and compare_sources:
        ext.extra_flags |= FLAG_SEARCH_TILES
        warm_up()
        t0 = time.perf_counter()
        for _ in range(steps):
            outs_search = ext.merged_spmv_launch(*args)
        torch.cuda.synchronize()
        ms_per_step_search = (time.perf_counter() - t0) * 1e3 / steps
        ext.extra_flags &= ~FLAG_SEARCH_TILES
        for o, r in zip(outs, outs_search):
            assert torch.equal(o, r), "launch that searched every boundary differs from a launch that confirmed the table"
    # ... and with the table taken on the caller's word, without the confirmation
    ms_per_step_reuse = None
    if ext.signature["has_reducer"] and compare_sources:
        ext.reuse_tiles = True
        warm_up()   # the launches one by one above let the clocks drop again
        t0 = time.perf_counter()
        for _ in range(steps):
            outs_reuse = ext.merged_spmv_launch(*args)
        torch.cuda.synchronize()
        ms_per_step_reuse = (time.perf_counter() - t0) * 1e3 / steps
        ext.reuse_tiles = False
        for o, r in zip(outs, outs_reuse):
            assert torch.equal(o, r), "launch with a reused tile table differs from a full launch"

    # the dominant kernel alone: HIP events attached to its dispatch inside the library, on the launch stream.
    # Every timed launch is issued between two untimed ones, so that the kernel runs in a busy stream as it
    # does in the K-step region (reading its events back idles the GPU for a moment).
    def kernel_series():
        warm_up()
        series = []
        for _ in range(steps):
            ext.merged_spmv_launch(*args)
            ext.time_kernel = True
            ext.merged_spmv_launch(*args)
            ext.time_kernel = False
            ext.merged_spmv_launch(*args)
            series.append(ext.last_kernel_ms())
        return series
    kernel_ms = kernel_series()
    kernel_ms_mean = sum(kernel_ms) / len(kernel_ms)
    kernel_ms.sort()
    # the same kernel in launches that search every boundary first (it then only reads the table)
    kernel_ms_search = None
    if ext.signature["has_reducer"] and compare_sources:
        ext.extra_flags |= FLAG_SEARCH_TILES
        series = kernel_series()
        ext.extra_flags &= ~FLAG_SEARCH_TILES
        kernel_ms_search = sum(series) / len(series)

    dtype = str(next(iter(w.tensors.values())).dtype)
    machine = None
    if calibrate:
        write_bytes = sum(o.numel() * o.element_size() for o in (outs or ()))
        machine = machine_mix_rate(ext, w, dtype, write_bytes)
    policy = ext.signature["policy"]
    flat = not ext.signature["has_reducer"]
    result = {
        "workload": w.name, "graph": w.graph, "dtype": dtype,
        "ne": int(w.ne), "num_rows": int(w.num_rows), "algorithmic_bytes": int(w.algorithmic_bytes),
        "flops": int(w.flops), "ms_per_step": ms_per_step,
        **({"ms_per_step_median_of_regions": region_ms[len(region_ms) // 2], "regions": len(region_ms)}
           if len(region_ms) > 1 else {}),
        "step_ms_median": step_ms[len(step_ms) // 2], "step_ms_min": step_ms[0],
        "kernel": "flex::flat_kernel" if flat else "flex::reduce_kernel",
        "kernel_ms": kernel_ms_mean, "kernel_ms_median": kernel_ms[len(kernel_ms) // 2], "kernel_ms_min": kernel_ms[0],
        "gbs": w.algorithmic_bytes / ms_per_step / 1e6, "kernel_gbs": w.algorithmic_bytes / kernel_ms_mean / 1e6,
        "edges_per_s": w.ne / ms_per_step * 1e3, "gflops": w.flops / ms_per_step / 1e6,
        "policy": policy, "policy_tag": f"{policy['block']}x{policy['ipt'][dtype]}",
        "seed": int(w.seed),
    }
    if library:
        result["library"] = library
        result["library_variant"] = ext.variant   # tuning switches and tile-shape override the file was built with
    if machine:
        result["machine"] = machine
    if ms_per_step_search is not None:
        result["ms_per_step_search_every_launch"] = ms_per_step_search
        result["gbs_search_every_launch"] = w.algorithmic_bytes / ms_per_step_search / 1e6
        result["kernel_ms_search_every_launch"] = kernel_ms_search
    if ms_per_step_reuse is not None:
        result["ms_per_step_tile_reuse"] = ms_per_step_reuse
        result["gbs_tile_reuse"] = w.algorithmic_bytes / ms_per_step_reuse / 1e6
    result["output_kinds"] = [o["kind"] for o in ext.signature["outputs"]]
    return result, [o.cpu().numpy() for o in outs]


def cpu_leg(w, result, outs, cpu_runs):
    """CPU leg, run after every GPU timing is done (its OpenMP threads would otherwise disturb the
    launch thread): times the oracle on the same inputs and checks the GPU outputs against it with the
    criterion of oracle/parity.py (row by row; every term of the allowance is the row's own)."""
    import numpy as np

    from flexspmv_amd import graphs
    if cpu_runs <= 0:
        return result
    from oracle.parity import FLOOR_ULPS, MOVE_FACTOR, aggregator_bounds, reducer_row_scales, row_excess
    from oracle.runner import run_oracle
    T = host_threads()
    ir = graphs.get(w.graph)
    ref = None
    times = []
    for i in range(cpu_runs + 1):
        c0 = time.perf_counter()
        ref, _ = run_oracle(ir, w.tensors, w.row_end_offsets, w.num_rows, w.num_cols, T)
        if i > 0:
            times.append(time.perf_counter() - c0)
    times.sort()
    cpu_ms = times[len(times) // 2] * 1e3
    tol = 1e-5 if result["dtype"] == "float32" else 1e-12
    scales = reducer_row_scales(ir, w.tensors, w.row_end_offsets, w.num_cols, T) if w.row_end_offsets is not None else {}
    # worst = the largest |difference| as a multiple of what the criterion allows (<= 1: within the tolerance)
    worst, fine_ok, aggregators = 0.0, True, {}
    centre = "oracle_" + DTYPE_TAG[result["dtype"]].replace("f", "fp")
    for i, (o, r) in enumerate(zip(outs, ref)):
        agg = aggregator_bounds(ir, w.tensors, w.row_end_offsets, w.num_rows, w.num_cols, i, tol)
        if agg is not None:
            # float32 aggregators: the reference's own sequential float32 sum drifts from the exact sum by far more
            # than the tolerance, so the centre is the oracle in float64; the distances to the float32 oracle at
            # this run's thread count and at 256 threads (shortest chains) are reported beside it
            centre = "oracle_fp32 for reducer outputs, oracle_fp64 for aggregator outputs"
            o64 = o.astype(np.float64)
            size = max(float(np.abs(agg["centre"]).max()), 1e-300)
            to_centre = float(np.abs(o64 - agg["centre"]).max()) / size
            to_fine = float(np.abs(o64 - agg["fine"].astype(np.float64)).max())
            fine_ok &= to_fine <= agg["bound_fine"]
            worst = max(worst, to_centre / tol)
            aggregators[ir.outputs[i]["name"]] = {
                "rel_diff_vs_fp64_oracle": to_centre,
                f"rel_diff_vs_fp32_oracle_{T}_threads": float(np.abs(o64 - r.astype(np.float64)).max()) / size,
                "rel_diff_vs_fp32_oracle_256_threads": to_fine / size,
                "bound_vs_fp32_oracle_256_threads": agg["bound_fine"] / size,
                "fp32_oracle_vs_fp64_oracle": float(np.abs(r.astype(np.float64) - agg["centre"]).max()) / size}
        elif i in scales:
            worst = max(worst, float(row_excess(o, r, tol, *scales[i]).max()))
        elif o.dtype.kind == "i":
            worst = max(worst, 0.0 if np.array_equal(o, r) else float("inf"))
        else:
            r64 = r.astype(np.float64)
            worst = max(worst, float(np.abs(o.astype(np.float64) - r64).max()) / max(float(np.abs(r64).max()), 1e-300) / tol)
    result["cpu"] = {"ms": cpu_ms, "gbs": w.algorithmic_bytes / cpu_ms / 1e6, "threads": T, "runs": cpu_runs,
                     "max_rel_diff_vs_gpu": worst * tol, "tolerance": tol,
                     "parity_ok": bool(worst <= 1.0) and fine_ok, "parity_centre": centre,
                     "parity_scale": "per row: max(|reference|, sum of |contributions| of the row); floor per row: "
                                     f"{FLOOR_ULPS} ulp of the row's largest contribution + {MOVE_FACTOR} x what moves of the "
                                     "inputs by an ulp or two change in the row's contributions; aggregators: |reference|"}
    if aggregators:
        result["cpu"]["float32_aggregators"] = aggregators
    return result


def roofline_of(r):
    # the traffic table holds the shipped libraries' counters; a variant given with --library has its own
    traffic = None if r.get("library") else measured_traffic(r["workload"], r["kernel"], r["policy_tag"])
    out = {"bound": "hbm", "achieved": r["kernel_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "frac": r["kernel_gbs"] / HBM_PEAK_GBS, "traffic": traffic["bytes"] if traffic else None,
           "kernel": r["kernel"], "kernel_ms": r["kernel_ms"], "kernel_ms_median": r["kernel_ms_median"],
           "kernel_ms_min": r["kernel_ms_min"], "launches": None}
    if traffic:
        out["traffic_source"] = traffic["source"]
    if r.get("kernel_ms_search_every_launch"):
        # the kernel of a launch that ran a search first does not confirm the table: its own work without that
        out["kernel_ms_search_every_launch"] = r["kernel_ms_search_every_launch"]
        out["frac_search_every_launch"] = r["algorithmic_bytes"] / r["kernel_ms_search_every_launch"] / 1e6 / HBM_PEAK_GBS
    if r.get("machine"):
        # the same bytes in the same tiles without the arithmetic: how much of the distance to the peak is the machine's
        out["same_mix_without_arithmetic"] = r["machine"]
        out["frac_of_same_mix"] = r["machine"]["ms"] * r["algorithmic_bytes"] / (
            r["machine"]["read_bytes"] + r["machine"]["write_bytes"]) / r["kernel_ms"]
    return out


def cpu_baseline_of(r):
    c = r["cpu"]
    return {"value": c["gbs"], "unit": "GB/s", "cores": c["threads"], "kind": "port",
            "sample": f"the whole workload ({r['workload']}), median of {c['runs']} runs after one warm-up, "
                      f"{c['ms']:.1f} ms per run",
            "ms": c["ms"], "parity_max_rel_diff": c["max_rel_diff_vs_gpu"], "parity_tolerance": c["tolerance"],
            "parity_ok": c["parity_ok"], "parity_centre": c["parity_centre"], "parity_scale": c["parity_scale"],
            **({"float32_aggregators": c["float32_aggregators"]} if "float32_aggregators" in c else {})}


def time_edge_list_preparation(w, steps):
    """The step in front of a launch, on this workload's edge list: ascending COO row ids -> row pointer, the
    stable sort by row of the shuffled list, and the permutation of one per-edge value array.  Bytes are
    algorithmic: ids read once, pointer written once; for the permutation index + value read, value written."""
    import torch
    from flexspmv_amd import formats
    ptr = torch.from_numpy(w.row_end_offsets).cuda()
    rows = torch.repeat_interleave(torch.arange(w.num_rows, device="cuda", dtype=torch.int32),
                                   (ptr[1:] - ptr[:-1]).to(torch.int64))
    ne, nr = rows.numel(), w.num_rows

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            e1.synchronize()
            best = min(best, e0.elapsed_time(e1) / reps)
        return best

    out = {}
    ms = timed(lambda: formats.coo_rows_to_csr_async(rows, nr), steps)
    got, findings = formats.coo_rows_to_csr_async(rows, nr)
    ok = bool(torch.equal(got, ptr.to(torch.int32))) and int(findings[0]) == 0
    b = 4 * ne + 4 * (nr + 1)
    out["coo_rows_to_csr"] = {"ms": ms, "algorithmic_bytes": b, "gbs": b / ms / 1e6, "frac_of_hbm_peak":
                              b / ms / 1e6 / HBM_PEAK_GBS, "matches_generator": ok}
    shuffled = rows[torch.randperm(ne, device="cuda")]
    ms = timed(lambda: formats.sort_edges_by_row(shuffled, nr), max(1, steps // 10))
    # radix sort, 8-bit digits over the bits of num_rows - 1; per digit the ids are read twice (counted, then moved
    # with their positions) and written once: 4 + 8 + 8 bytes per edge, the first digit 4 + 4 + 8 (positions implicit)
    digits = -(-max(1, (nr - 1).bit_length()) // 8)
    b = ne * (16 + 20 * (digits - 1))
    out["sort_edges_by_row"] = {"ms": ms, "edges_per_s": ne / ms * 1e3, "digits": digits, "algorithmic_bytes": b,
                                "gbs": b / ms / 1e6, "frac_of_hbm_peak": b / ms / 1e6 / HBM_PEAK_GBS,
                                "torch_stable_sort_ms": timed(lambda: torch.sort(shuffled, stable=True),
                                                              max(1, steps // 10))}
    _, perm = formats.sort_edges_by_row(shuffled, nr)
    vals = torch.from_numpy(next(v for v in w.tensors.values() if v.dtype.kind == "f" and v.shape[0] == ne)).cuda()
    dst = torch.empty_like(vals)
    ms = timed(lambda: formats.gather_rows(vals, perm, out=dst), max(1, steps // 5))
    b = ne * (4 + 2 * vals.element_size() * (vals.numel() // ne))
    line_traffic = ne * (4 + 128 + vals.element_size() * (vals.numel() // ne))   # a whole 128-byte line per random read
    out["gather_rows"] = {"ms": ms, "algorithmic_bytes": b, "gbs": b / ms / 1e6, "order": "random permutation",
                          "line_traffic_bytes": line_traffic, "line_traffic_gbs": line_traffic / ms / 1e6}
    # a permutation with locality: the edge list in column order (the transpose's row order)
    cols = next((torch.from_numpy(v).cuda() for k, v in w.tensors.items()
                 if k.endswith("_idx") and v.shape[0] == ne and not k.startswith("selector_row")), None)
    if cols is not None:
        _, perm_t = formats.sort_edges_by_row(cols, w.num_cols)
        ms = timed(lambda: formats.gather_rows(vals, perm_t, out=dst), max(1, steps // 5))
        out["gather_rows_transpose_order"] = {"ms": ms, "algorithmic_bytes": b, "gbs": b / ms / 1e6,
                                              "order": "edges sorted by column (stable)"}
    return out


def torch_sparse_comparison(w, reps: int = 10):
    """The same product by torch's own kernels, for SpMV workloads: `index_select` of x by the column index (the
    gather alone) and the sparse-CSR product the installed torch dispatches to its vendor library.  Microseconds
    per call, events around `reps` back-to-back calls."""
    import torch
    from flexspmv_amd import workloads as W
    from flexspmv_amd.binding import load_named
    names = load_named(w.graph, build_if_missing=False).param_names()
    col_name = next((n for n in ("selector_idx", "selector_col_idx") if n in names), None)
    if col_name is None or "vals" not in names or "x" not in names:
        return None
    args = W.launch_arguments(w, names, "cuda:0")
    x, cols, vals = (args[names.index(n)] for n in ("x", col_name, "vals"))
    row_ptr = args[names.index("row_end_offsets")]

    def us(call):
        call()
        torch.cuda.synchronize()
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        for _ in range(reps):
            call()
        t1.record()
        torch.cuda.synchronize()
        return round(t0.elapsed_time(t1) / reps * 1e3, 1)

    gathered = torch.empty(cols.numel(), dtype=x.dtype, device=x.device)
    out = {"unit": "us per call",
           "index_select_of_x_by_column": us(lambda: torch.index_select(x, 0, cols, out=gathered))}
    del gathered
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        matrix = torch.sparse_csr_tensor(row_ptr, cols, vals, size=(w.num_rows, w.num_cols))
    column = x.unsqueeze(1)
    if w.graph == "spmv_dot":
        out["sparse_csr_product_and_dot"] = us(lambda: torch.dot(x, (matrix @ column).squeeze(1)))
    else:
        out["sparse_csr_product"] = us(lambda: matrix @ column)
    del matrix
    torch.cuda.empty_cache()
    return out


def machine_rates(gib: int = 2, reps: int = 20):
    """TB/s of three library kernels on tensors of `gib` GiB (events around `reps` back-to-back calls)."""
    import torch
    n = gib << 27   # float64 elements
    src = torch.empty(n, dtype=torch.float64, device="cuda:0").fill_(1.0)
    dst = torch.empty_like(src)

    def rate(call, nbytes):
        call()
        torch.cuda.synchronize()
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        for _ in range(reps):
            call()
        t1.record()
        torch.cuda.synchronize()
        return round(nbytes / (t0.elapsed_time(t1) / reps * 1e-3) / 1e12, 3)

    one = n * 8
    out = {"tensor_bytes": one, "unit": "TB/s",
           "write_only_fill": rate(lambda: dst.fill_(1.0), one),
           "read_only_sum": rate(lambda: src.sum(), one),
           "read_write_1_to_1_add": rate(lambda: torch.add(src, 1.0, out=dst), 2 * one)}
    del src, dst
    # uniformly random 4-byte gathers (index_select, 2^26 int32 indices) from tables of several sizes
    count = 1 << 26
    gen = torch.Generator(device="cuda:0").manual_seed(3)
    gathered = torch.empty(count, dtype=torch.float32, device="cuda:0")
    out["random_gathers"] = {"unit": "T gathers/s", "indices": count}
    for table_bytes in (1 << 16, 1 << 22, 1 << 24, 1 << 26):
        table = torch.rand(table_bytes // 4, device="cuda:0")
        idx = torch.randint(0, table.numel(), (count,), device="cuda:0", dtype=torch.int32, generator=gen)
        out["random_gathers"][f"table_of_{table_bytes}_bytes"] = rate(
            lambda: torch.index_select(table, 0, idx, out=gathered), count)
        del table, idx
    del gathered
    torch.cuda.empty_cache()
    return out


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="poisson3d", choices=sorted(DEFAULT_SIZE))
    ap.add_argument("--size", type=int, default=None, help="grid edge / R-MAT scale / point count")
    ap.add_argument("--mtx", default=None, help="time SpMV on this MatrixMarket file instead of a generated workload "
                                                "(float64 y = A x)")
    ap.add_argument("--mtx-dot", action="store_true", help="with --mtx: the fused form y = A x and x . y")
    ap.add_argument("--others", default=None,
                    help="comma-separated workloads timed after the headline one and reported under other_workloads "
                         "(default: the other four when the headline is the default Poisson run; 'none' for none)")
    ap.add_argument("--all", action="store_true", help="time all the other four workloads (extra JSON key)")
    ap.add_argument("--cpu-runs", type=int, default=5, help="timed runs of the CPU baseline (0 = skip)")
    ap.add_argument("--default-launches-only", action="store_true",
                    help="skip the series that search every boundary on every launch and that take the tile table on "
                         "trust (a kernel trace then holds the default launches only)")
    ap.add_argument("--no-calibration", action="store_true",
                    help="skip the calibration kernel (the workload's reads and writes without arithmetic)")
    ap.add_argument("--library", default=None,
                    help="time this library file on the workload instead of the shipped one: a variant of the same "
                         "sub-graph with another tile shape or tuning switches, from python -m flexspmv_amd.build")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain elementwise copies (dst = src + 1) of 1 GiB, a kernel of known "
                         "traffic, to scale rocprofv3's FETCH_SIZE / WRITE_SIZE counters")
    ap.add_argument("--torch-sparse", action="store_true",
                    help="also time torch's own kernels on the headline workload, if it is an SpMV: index_select of x "
                         "by the column index and the sparse-CSR product (extra JSON key)")
    ap.add_argument("--machine-rates", action="store_true",
                    help="also time torch's fill, sum and dst = src + 1 on 2 GiB tensors and its index_select with random "
                         "indices: what this GPU gives a library's streaming and gathering kernels (extra JSON key)")
    ap.add_argument("--formats", action="store_true",
                    help="also time the edge-list preparation kernels on this workload's edge list (extra JSON key)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this path runs on one GPU; --gpus must be 1 (no multi-GPU figure exists for it)",
              file=sys.stderr)
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    from flexspmv_amd import workloads as W

    size = a.size if a.size is not None else DEFAULT_SIZE[a.workload]
    if a.mtx is not None:
        w = W.matrix_market_spmv(a.mtx, fused_dot=a.mtx_dot)
    else:
        w = W.WORKLOADS[a.workload](size)
    head, head_outs = time_workload(w, a.steps, a.warmup, library=a.library, calibrate=not a.no_calibration,
                                    compare_sources=not a.default_launches_only)
    torch.cuda.empty_cache()
    if a.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda:0").fill_(1.0)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)   # one elementwise kernel: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()
    rates = machine_rates() if a.machine_rates else None
    torch_sparse = torch_sparse_comparison(w) if a.torch_sparse else None
    if a.all:
        other_names = [n for n in ("rmat", "spring_mass", "shallow_water", "laplacian2d") if n != a.workload]
    elif a.others is not None:
        other_names = [n for n in a.others.split(",") if n and n != "none"]
    else:
        other_names = (["rmat", "shallow_water", "spring_mass", "laplacian2d"]
                       if (a.workload == "poisson3d" and a.mtx is None and a.size is None) else [])
    pending = []
    for name in other_names:
        wo = W.WORKLOADS[name](DEFAULT_SIZE[name])
        r, o = time_workload(wo, a.steps, a.warmup, calibrate=not a.no_calibration,
                             compare_sources=not a.default_launches_only)
        torch.cuda.empty_cache()
        pending.append((name, wo, r, o))
    head = cpu_leg(w, head, head_outs, a.cpu_runs)
    others = {}
    for name, wo, r, o in pending:
        r = cpu_leg(wo, r, o, min(a.cpu_runs, 3))
        entry = {k: r[k] for k in ("workload", "graph", "dtype", "ne", "num_rows", "algorithmic_bytes", "seed", "policy",
                                   "ms_per_step", "ms_per_step_median_of_regions", "regions", "step_ms_median",
                                   "step_ms_min", "gbs", "edges_per_s", "gflops",
                                   "ms_per_step_search_every_launch", "gbs_search_every_launch",
                                   "ms_per_step_tile_reuse", "gbs_tile_reuse") if k in r}
        entry["pct_of_hbm_peak"] = 100.0 * r["gbs"] / HBM_PEAK_GBS
        entry["roofline"] = roofline_of(r)
        entry["roofline"]["launches"] = a.steps
        if "cpu" in r:
            entry["cpu_baseline"] = cpu_baseline_of(r)
        if name in WORKLOAD_NOTES:
            entry["note"] = WORKLOAD_NOTES[name]
        others[name] = entry

    parity_ok = all(r.get("cpu", {}).get("parity_ok", True) for r in [head] + [p[2] for p in pending])
    line = {
        "metric": "fused SpMV effective HBM GB/s (% of MI355X peak) + edges/sec, 1 GPU",
        "value": head["gbs"] if parity_ok else None,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": DTYPE_TAG[head["dtype"]],
        "data": "synthetic",
        "config": {"workload": f"{head['workload']} " + ("fused y=A*x and x.y" if head["graph"] == "spmv_dot"
                                                        else "y=A*x" if head["graph"] == "csr_spmv" else "step")
                               + f" ({head['graph']})", "ne": head["ne"],
                   "num_rows": head["num_rows"], "algorithmic_bytes": head["algorithmic_bytes"],
                   "policy": head["policy"], "seed": head["seed"]},
        **({k: head[k] for k in ("ms_per_step_median_of_regions", "regions") if k in head}),
        "step_ms_median": head["step_ms_median"],
        "step_ms_min": head["step_ms_min"],
        "pct_of_hbm_peak": 100.0 * head["gbs"] / HBM_PEAK_GBS,
        "edges_per_s": head["edges_per_s"],
        "gflops": head["gflops"],
        "roofline": roofline_of(head),
    }
    line["roofline"]["launches"] = a.steps
    if a.workload in WORKLOAD_NOTES and a.mtx is None:
        line["config"]["note"] = WORKLOAD_NOTES[a.workload]
    if a.library:
        line["config"]["library"] = a.library   # not the shipped library: a variant built for a measurement
        line["config"]["library_variant"] = head["library_variant"]
    if "ms_per_step_search_every_launch" in head:
        line["tile_table"] = {
            "headline": "every block takes its tile's boundaries from the table the launch before left in the scratch and "
                        "confirms them against this launch's row pointer (three row ends per boundary, fetched with the "
                        "tile); the K timed launches follow the warm-up on the same matrix, so no search runs in them",
            "search_every_launch": {"ms_per_step": head["ms_per_step_search_every_launch"],
                                    "value": head["gbs_search_every_launch"], "unit": "GB/s",
                                    "note": "FLEXSPMV_FLAG_SEARCH_TILES: every boundary searched on every launch, as the "
                                            "reference does (a search kernel in front of the reducer)"},
            "taken_on_trust": {"ms_per_step": head["ms_per_step_tile_reuse"], "value": head["gbs_tile_reuse"],
                               "unit": "GB/s", "note": "FLEXSPMV_FLAG_REUSE_TILES: the table used without the confirmation"}}
    if "cpu" in head:
        line["cpu_baseline"] = cpu_baseline_of(head)
    if others:
        line["other_workloads"] = others
    if rates is not None:
        line["machine_rates"] = rates
    if torch_sparse is not None:
        line["torch_sparse"] = torch_sparse
    if a.formats:
        line["edge_list_preparation"] = time_edge_list_preparation(w, a.steps)
    if not parity_ok:
        line["error"] = "GPU result outside the parity tolerance: value withheld"
    print(json.dumps(line))
    return 0 if parity_ok else 1


if __name__ == "__main__":
    sys.exit(main())
