#!/usr/bin/env python3
"""Benchmark of the hipDMA transfer patterns on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME[,NAME...]] [--no-cpu-baseline]

A step is one launch of the CudaDMAStrided tile-transpose kernel over the whole 16384 x 16384 float32
matrix (benchmark config 2, the configuration the metric is quoted on).  The inputs of every pattern of the run
are generated on the device first, so every timed region starts with its inputs resident in HBM; the headline is
then timed exactly as the command line says (--warmup launches, then --steps timed ones).  The other HBM-bound patterns (sequential copy, indirect gather, halo stencil), the scatter
in the opposite direction and the GEMM are timed the same way (HIP events on the launch stream) and reported
under "patterns" / "gemm".  The sequential copy and the gather are each reported twice: at the size the
configuration names (64 MiB buffer, 512 MiB table: both working sets are helped by the 256 MB Infinity Cache)
and at a size that is not (1 GiB buffer, 4 GiB table).  "yardsticks" holds what read-only, write-only and
copy-shaped streams and the vendor's own device-to-device copy reach on the same 1 GiB buffers in the same
run; roofline.ceiling is the best read + write yardstick of the run.  Every row of "patterns" also carries a
"ceiling" of its own: what a kernel without LDS and without a DMA object reaches in the same run on the same buffers with
the pattern's own addresses (the gather's index list, the scatter's permutation, a plain copy for the sequential and
strided patterns and, scaled by the stencil's measured traffic, for the halo), and "settle_ms": the wall time of untimed
launches in front of the timed ones.  The headline row "strided" is timed exactly as the command line says (--warmup
launches, then --steps timed ones); "strided_settled" is the same kernel under the policy of the other rows.
Counter-derived fields (HBM traffic per launch, matrix-core occupancy) come from profiles/counters.json, which
`python -m cudadma_amd.profile_summary` writes from rocprofv3 output.  One JSON line goes to stdout; progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0           # MI355X published HBM3E bandwidth
MFMA_PEAK_TFLOPS = 2500.0       # MI355X published dense bf16 rate
SETTLE_MS = 30.0                # wall time of untimed warm-up for the secondary patterns
STRIDED_VARIANT = 0             # cudadma_strided_transpose variant timed as the headline: the library's choice (three DMA + one compute wavefront)
COUNTERS_JSON = os.path.join(ROOT, "profiles", "counters.json")

# name -> (kernel the pattern launches, as rocprofv3 names it; used by cudadma_amd.profile_summary)
PATTERN_KERNELS = {
    "strided": "transpose_split<3, 1, 1, false>",
    "strided_settled": "transpose_split<3, 1, 1, false>",
    "sequential_read_probe": "perf_manual<2, 4>",
    "strided_even_split": "transpose_single<true, true>",
    "strided_double_buffered_lds": "transpose_double_lds<3, 1>",
    "strided_two_lds_tiles": "transpose_manual_double<272, false>",
    "sequential": "copy_manual_double<4>",
    "sequential_hbm": "copy_single<true, false>",
    "gather": "gather_manual<(anonymous namespace)::RowsumConsumer, 2, true>",
    "gather_hbm": "gather_manual<(anonymous namespace)::RowsumConsumer, 2, true>",
    "scatter": "scatter_manual<4>",
    "halo": "stencil_ws_vec4<2, 8>",
    "halo_handshake": "stencil_ws_vec4<0, 8>",
    "halo_wide_tiles": "stencil_ws_vec4<2, 8>",          # the same template in the translation unit compiled for 64 x 16 tiles
    "gemm": "gemm_bf16_all_direct_a64",
    "gemm_warp_specialised": "gemm_bf16_ws_direct4_a64",
}


def log(msg):
    print(msg, file=sys.stderr, flush=True)


def load_counters():
    """profiles/counters.json or an empty record (the counter-derived fields are then null)."""
    try:
        with open(COUNTERS_JSON) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


def time_launches(fn, steps, warmup, settle_ms=0.0):
    """Average milliseconds per launch, HIP events on the launch stream around `steps` launches.
    `settle_ms` > 0 keeps the untimed warm-up going for that much wall time (used for the
    secondary patterns: the first launches after an allocation phase run up to 25 % slow)."""
    import torch
    t0 = time.perf_counter()
    done = 0
    while done < warmup or (time.perf_counter() - t0) * 1e3 < settle_ms:
        fn()
        done += 1
        if done % 8 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return start.elapsed_time(stop) / steps, wall_ms / steps


def _median_time(fn, budget_s, min_reps=3, max_reps=200):
    fn()                                             # warm-up + first touch of the output
    times = []
    t_all = time.perf_counter()
    while len(times) < min_reps or (len(times) < max_reps and time.perf_counter() - t_all < budget_s):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return sorted(times)[len(times) // 2], len(times)


def cpu_baselines(budget_s=15.0):
    """The oracle's OpenMP implementation of each pattern on this machine's host cores, on the full
    configurations (inputs generated in parallel, so first touch is spread over the cores); bytes counted as for
    the GPU figures.  Returns the headline object (strided transpose) and a per-pattern dictionary."""
    import numpy as np
    from tests import oracle_lib as ol
    from tests.oracle_lib import ptr
    O = ol.load()
    cores = O.oracle_num_threads()
    per = budget_s / 5
    out = {}

    n = 16384                                        # config 2 whole: 1 GiB in, 1 GiB out
    a = ol.uniform(n * n, 1002).reshape(n, n)
    t = np.empty_like(a)
    med, reps = _median_time(lambda: O.oracle_transpose(ptr(a), ptr(t), n), per)
    out["strided"] = {"GB/s": round(2.0 * n * n * 4 / med / 1e9, 2),
                      "sample": f"oracle_transpose (256x256 tiles, 16x16 blocks through a local buffer) of the full {n}x{n} float32 matrix, median of {reps}"}
    del a, t

    m = 64 * 1024 * 1024 // 4                        # config 1 whole: 64 MiB (resident in the host caches) ...
    src = ol.uniform(m, 1001)
    dst = np.empty_like(src)
    med, reps = _median_time(lambda: O.oracle_copy(ptr(src), ptr(dst), m), per / 2)
    out["sequential"] = {"GB/s": round(2.0 * m * 4 / med / 1e9, 2),
                         "sample": f"oracle_copy of the full 64 MiB buffer ({64 // cores if cores else 64} MiB per thread: helped by the host caches), median of {reps}"}
    del src, dst
    m = 1024 * 1024 * 1024 // 4                      # ... and the 1 GiB buffer of the sequential_hbm row
    src = ol.uniform(m, 1001)
    dst = np.empty_like(src)
    med, reps = _median_time(lambda: O.oracle_copy(ptr(src), ptr(dst), m), per / 2)
    out["sequential_hbm"] = {"GB/s": round(2.0 * m * 4 / med / 1e9, 2),
                             "sample": f"oracle_copy of a 1 GiB buffer, median of {reps}"}
    del src, dst

    recs, n_idx = 4 * 1024 * 1024, 32 * 1024 * 1024   # config 3 whole: 512 MiB table, 32 Mi indices
    table = ol.uniform(recs * 32, 1003)
    idx = ol.indices(n_idx, recs, 1003)
    sums = np.empty(n_idx // 32 * 32, dtype=np.float32)
    med, reps = _median_time(lambda: O.oracle_gather_rowsum(ptr(table), ptr(idx), ptr(sums), n_idx, 32, 32), per)
    out["gather"] = {"GB/s": round((n_idx * 132 + sums.size * 4) / med / 1e9, 2),
                     "sample": f"oracle_gather_rowsum over the full 512 MiB table with all {n_idx} indices, median of {reps}"}
    del table, idx, sums

    log2_recs = 22                                   # the whole scatter: 512 MiB of records, 4 Mi indices
    n_rec = 1 << log2_recs
    records = ol.uniform(n_rec * 32, 1006)
    perm = ol.permutation(log2_recs, 1006)
    table = np.empty(n_rec * 32, dtype=np.float32)
    med, reps = _median_time(lambda: O.oracle_scatter_copy(ptr(records), ptr(perm), ptr(table), n_rec, 32), per)
    out["scatter"] = {"GB/s": round(n_rec * 260 / med / 1e9, 2),
                      "sample": f"oracle_scatter_copy of {n_rec} records of 128 B by a permutation, median of {reps}"}
    del records, perm, table

    g, p = 512, 4                                    # config 4 whole
    grid = ol.uniform((g + 2 * p) ** 3, 1004)
    res = np.empty(g ** 3, dtype=np.float32)
    med, reps = _median_time(lambda: O.oracle_stencil25(ptr(grid), ptr(res), g, g, g, p), per)
    out["halo"] = {"GB/s": round(2.0 * g ** 3 * 4 / med / 1e9, 2),
                   "sample": f"oracle_stencil25 on the full {g}^3 float32 grid, median of {reps}"}

    del grid, res

    dim, rows = 4096, 1024                           # config 5, a quarter of the rows of C (the loop nest is the same for every row)
    ga = np.empty(rows * dim, dtype=np.uint16)
    gb = np.empty(dim * dim, dtype=np.uint16)
    gc = np.empty(rows * dim, dtype=np.float32)
    O.oracle_fill_normal_bf16(ptr(ga), ga.size, 1005)
    O.oracle_fill_normal_bf16(ptr(gb), gb.size, 2005)
    t0 = time.perf_counter()
    O.oracle_gemm_bf16(ptr(ga), ptr(gb), ptr(gc), rows, dim, dim)
    dt = time.perf_counter() - t0
    out["gemm"] = {"TFLOP/s": round(2.0 * rows * dim * dim / dt / 1e12, 4),
                   "sample": f"oracle_gemm_bf16 (fp32 products of the bf16 inputs, ascending k) on the first {rows} of the {dim} rows of C "
                             f"of the {dim}^3 problem, one repetition of {dt:.1f} s"}

    head = {"value": out["strided"]["GB/s"], "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "OpenMP " + out["strided"]["sample"]}
    return head, out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-core baseline leg")
    ap.add_argument("--only", default="", help="comma-separated pattern names to run besides the headline "
                    "(for profiling one kernel at a time); 'strided' alone runs the headline only")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (the DMA objects live inside one kernel on one "
                 "device; there is no multi-GPU path to time). Use --gpus 1.")

    import torch
    import cudadma_amd as cd
    from cudadma_amd import workloads as wl

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the hipDMA kernels have no CPU path")
    dev = torch.device("cuda:0")
    cd.lib()
    steps, warmup = args.steps, args.warmup
    only = set(x for x in args.only.split(",") if x)
    want = lambda name: not only or name in only
    counters = load_counters()
    traffic = lambda name: (counters.get("patterns", {}).get(name) or {}).get("traffic_bytes")
    patterns, yardsticks = {}, {}
    cus = torch.cuda.get_device_properties(0).multi_processor_count

    def report(table, name, ms, nbytes, note, bound="hbm", settle_ms=SETTLE_MS, launches=None):
        gbs = nbytes / ms / 1e6
        row = {"GB/s": round(gbs, 1), "frac_of_peak": round(gbs / HBM_PEAK_GBS, 4), "ms": round(ms, 4),
               "algorithmic_bytes": nbytes, "bound": bound, "settle_ms": settle_ms,
               "timed_launches": launches if launches is not None else steps, "workload": note}
        if table is patterns:
            row["kernel"] = PATTERN_KERNELS.get(name)
            row["traffic_bytes_from_counters"] = traffic(name)
        table[name] = row
        log(f"{name:24s} {ms:9.4f} ms  {gbs:8.1f} GB/s  {100 * gbs / HBM_PEAK_GBS:5.1f}% of peak   {note}")

    def best_shape(launch, choices, nbytes, label, note):
        """The fastest of a few launch shapes of a yardstick; launch(choice) returns the function to time."""
        best = None
        for choice in choices:
            ms, _ = time_launches(launch(choice), max(10, steps // 2), 5, 10.0)
            if best is None or ms < best[0]:
                best = (ms, choice)
        report(yardsticks, label, best[0], nbytes, note.format(best=best[1], tried=len(choices)), settle_ms=10.0, launches=max(10, steps // 2))

    # ---- config 2: strided tile transpose (headline) ----
    # One allocation holds the source and, exactly 1 GiB behind it, the destination of every 1 GiB + 1 GiB stream of
    # this run: the rate of a linear copy depends on the distance between its two buffers (0.350 to 0.440 ms for the
    # same kernel as the distance varies modulo 64 MiB; the transposition does not care), and two separate
    # allocations land wherever the allocator, or a profiler loaded into the process, leaves room.
    n = 16384
    setup_start, setup_stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    setup_start.record()
    pool = torch.empty(2 * n * n, dtype=torch.float32, device=dev)
    src = wl.fill_uniform(pool[:n * n], 1002).view(n, n)
    dst = pool[n * n:].view(n, n)
    # The inputs of every other pattern of the run are generated here as well, before anything is timed: every timed
    # region then starts with its inputs resident in HBM, and the device has left its idle state (the shader clock dips
    # from 2.42 to 2.13-2.25 GHz between 1.5 and 8 ms after work begins on an idle device) by the time the first one starts.
    inputs = {}
    if want("sequential"):
        m = 64 * 1024 * 1024 // 4
        s_src = wl.fill_uniform(torch.empty(m, dtype=torch.float32, device=dev), 1001)
        inputs["sequential"] = (s_src, torch.empty_like(s_src))
    n_idx = 32 * 1024 * 1024
    for name, recs in (("gather", 4 * 1024 * 1024), ("gather_hbm", 32 * 1024 * 1024)):
        if want(name):
            inputs[name] = (wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, dtype=torch.float32, device=dev), 1003),
                            wl.fill_indices(torch.empty(n_idx, dtype=torch.int32, device=dev), recs, 1003),
                            torch.empty(n_idx // wl.RECS_PER_TILE * wl.REC_FLOATS, dtype=torch.float32, device=dev))
    if want("scatter"):
        recs = 4 * 1024 * 1024
        inputs["scatter"] = (wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, dtype=torch.float32, device=dev), 1006),
                             wl.fill_permutation(torch.empty(recs, dtype=torch.int32, device=dev), 1006),
                             torch.empty(recs * wl.REC_FLOATS, dtype=torch.float32, device=dev))
    if want("halo") or want("halo_handshake") or want("halo_wide_tiles"):
        g, p = 512, 2 * wl.STENCIL_RADIUS
        inputs["halo"] = (wl.fill_uniform(torch.empty((g + p) ** 3, dtype=torch.float32, device=dev), 1004).view(g + p, g + p, g + p),
                          torch.empty((g, g, g), dtype=torch.float32, device=dev))
    if want("gemm") or want("gemm_warp_specialised"):
        dim = 4096
        inputs["gemm"] = (wl.fill_normal_bf16(torch.empty((dim, dim), device=dev, dtype=torch.bfloat16), 1005),
                          wl.fill_normal_bf16(torch.empty((dim, dim), device=dev, dtype=torch.bfloat16), 2005),
                          torch.empty((dim, dim), device=dev, dtype=torch.float32))
    setup_stop.record()
    torch.cuda.synchronize()
    setup_ms = setup_start.elapsed_time(setup_stop)
    log(f"inputs generated in {setup_ms:.1f} ms of device time")
    strided_ms, strided_wall_ms = time_launches(lambda: wl.strided_transpose(src, dst, STRIDED_VARIANT), steps, warmup)
    strided_bytes = 2 * n * n * 4
    strided_note = ("CudaDMAStrided 64x256B tiles of a 16384^2 f32 matrix, transposed out: one LDS tile, the next tile in the DMA "
                    "wavefronts' registers (the double buffer is LDS + registers), one workgroup of three DMA wavefronts and one "
                    "compute wavefront per compute unit")
    report(patterns, "strided", strided_ms, strided_bytes, strided_note + f"; timed as the command line says: {warmup} untimed launches, "
           f"then {steps} timed ones, right after the inputs of the whole run were generated ({setup_ms:.0f} ms of device time)", settle_ms=0.0)
    patterns["strided"]["device_ms_of_input_generation_before"] = round(setup_ms, 1)
    if want("strided_settled"):
        ms, _ = time_launches(lambda: wl.strided_transpose(src, dst, STRIDED_VARIANT), steps, warmup, SETTLE_MS)
        report(patterns, "strided_settled", ms, strided_bytes, "the kernel of the strided row under the policy of the rows below")
    if want("strided_even_split"):
        ms, _ = time_launches(lambda: wl.strided_transpose(src, dst, 1), steps, warmup, SETTLE_MS)
        report(patterns, "strided_even_split", ms, strided_bytes, "the same kernel shape with two DMA and two compute wavefronts (128 + 128 threads)")
    if want("strided_double_buffered_lds"):
        ms, _ = time_launches(lambda: wl.strided_transpose(src, dst, wl.TRANSPOSE_DOUBLE_LDS_VARIANT), steps, warmup, SETTLE_MS)
        report(patterns, "strided_double_buffered_lds", ms, strided_bytes,
               "the double buffer in LDS: two LDS tiles with a guard each, filled in turn by one CudaDMAStrided object, the next tile in "
               "the DMA wavefronts' registers (one tile of loads in flight), three DMA wavefronts + one compute wavefront, one workgroup "
               "per compute unit")
    if want("strided_two_lds_tiles"):
        ms, _ = time_launches(lambda: wl.strided_transpose(src, dst, wl.TRANSPOSE_TWO_LDS_TILES_VARIANT), steps, warmup, SETTLE_MS)
        report(patterns, "strided_two_lds_tiles", ms, strided_bytes,
               "the same transposition with two LDS tiles and two CudaDMAStrided objects (manual double buffering in LDS: two tiles "
               "of loads in flight, four workgroups per compute unit)")
    # ---- yardsticks on the same two 1 GiB buffers: the plain copy used to calibrate the counters, the vendor's
    # copy, and read-only / write-only / copy streams each at the best of a few launch shapes ----
    flat_src, flat_dst = src.view(-1), dst.view(-1)
    if want("yardsticks") or want("plain_copy"):
        ms, _ = time_launches(lambda: wl.plain_copy(src, dst), steps, warmup, SETTLE_MS)
        report(yardsticks, "plain_copy", ms, strided_bytes, "grid-stride dwordx4 copy of 1 GiB at eight workgroups per compute "
               "unit, no LDS, no DMA object (the kernel the traffic counters are calibrated against)")
    if want("yardsticks"):
        ms, _ = time_launches(lambda: wl.probe_memory("vendor_copy", flat_src, flat_dst, 1), steps, warmup, SETTLE_MS)
        report(yardsticks, "vendor_copy", ms, strided_bytes, "hipMemcpyDtoDAsync of 1 GiB")

        def stream_shapes(modes, s_, d_, shapes):
            return ([(mode, wg) for mode in modes for wg in shapes],
                    lambda c: (lambda: wl.probe_memory(c[0], s_, d_, int(cus * c[1]))))
        stream_note = "{best[0]} stream over 1 GiB, grid-stride dwordx4, best of {tried} (cache hint, launch shape) pairs: {best[1]} workgroups per compute unit"
        choices, launch = stream_shapes(("read", "read_nontemporal"), flat_src, None, (1, 1.5, 2, 3, 4))
        best_shape(launch, choices, strided_bytes // 2, "read_only", stream_note)
        choices, launch = stream_shapes(("write", "write_nontemporal"), None, flat_dst, (0.5, 1, 2, 4))
        best_shape(launch, choices, strided_bytes // 2, "write_only", stream_note)
        choices, launch = stream_shapes(("copy", "copy_nontemporal"), flat_src, flat_dst, (1, 2, 4, 8))
        best_shape(launch, choices, strided_bytes, "copy_best_shape", stream_note)
        # the two halves of the transposition alone, with its own addresses in its own order
        sink = torch.empty(8 * cus * 4, dtype=torch.float32, device=dev)
        best_shape(lambda wg: (lambda: wl.probe_pattern("tile_read", src, None, sink, int(cus * wg))), (1, 1.5, 2, 3, 4), strided_bytes // 2,
                   "strided_reads_alone", "the source tiles of the transposition (64 rows x 256 B, rows 64 KiB apart) read in its tile order, "
                   "nothing written; best of {tried} launch shapes: {best} workgroups per compute unit")
        best_shape(lambda wg: (lambda: wl.probe_pattern("tile_write", None, None, dst, int(cus * wg))), (0.5, 1, 1.5, 2, 3), strided_bytes // 2,
                   "strided_writes_alone", "the destination tiles of the transposition written in its tile order, nothing read; best of "
                   "{tried} launch shapes: {best} workgroups per compute unit")
        del sink
    del src, dst, flat_src, flat_dst

    # ---- config 1: sequential copy in 16 KiB tiles: the 64 MiB of the configuration, and 1 GiB ----
    if want("sequential"):
        m = 64 * 1024 * 1024 // 4
        s_src, s_dst = inputs.pop("sequential")
        ms, _ = time_launches(lambda: wl.sequential_copy(s_src, s_dst, 0), max(steps, 50), warmup, SETTLE_MS)
        report(patterns, "sequential", ms, 2 * m * 4, "CudaDMASequential 16 KiB tiles of the configuration's 64 MiB f32 buffer: the "
               "128 MiB working set stays in the 256 MB Infinity Cache from launch to launch, so this is a cache-assisted rate, "
               "not an HBM rate", bound="infinity cache + hbm", launches=max(steps, 50))
        if want("yardsticks"):
            best_shape(lambda c: (lambda: wl.probe_memory(c[0], s_src, s_dst, int(cus * c[1]))),
                       [(mode, wg) for mode in ("copy", "copy_nontemporal") for wg in (2, 4, 8)], 2 * m * 4, "copy_best_shape_64MiB",
                       "{best[0]} stream over the same 64 MiB buffers (cache-assisted like the sequential row), best of {tried} "
                       "(cache hint, launch shape) pairs: {best[1]} workgroups per compute unit")
        del s_src, s_dst
    if want("sequential_hbm"):
        m = 1024 * 1024 * 1024 // 4
        s_src = wl.fill_uniform(pool[:m], 1001)
        s_dst = pool[m:]
        ms, _ = time_launches(lambda: wl.sequential_copy(s_src, s_dst, 0), steps, warmup, SETTLE_MS)
        report(patterns, "sequential_hbm", ms, 2 * m * 4, "the same entry point on a 1 GiB buffer (2 GiB working set, eight times the Infinity Cache): one LDS tile, the "
               "next tile in the DMA wavefronts' registers, two workgroups per compute unit, streaming loads and non-temporal stores; "
               "destination exactly 1 GiB behind the source")
        del s_src, s_dst
    if want("sequential_read_probe"):
        # the reference's own metric (src/perf/sequential/perf_sequential.cu:354-361): bytes read into LDS per second, nothing written
        m = 1024 * 1024 * 1024 // 4
        s_src = pool[:m]
        groups, elmt = 2 * cus, 16 * 1024
        loops = (m * 4) // (groups * elmt)
        run = lambda: wl.perf_sequential(s_src, elmt, 4, wl.BUFFERING_MANUAL, loops, groups, None, wl.LOAD_CACHE_STREAMING, wl.STORE_LDS)
        nbytes = run()
        ms, _ = time_launches(run, steps, warmup, SETTLE_MS)
        report(patterns, "sequential_read_probe", ms, nbytes, "the reference's read-bandwidth probe on CudaDMASequential: 1 GiB read into LDS in "
               "16 KiB elements and dropped, four DMA wavefronts + one compute wavefront per workgroup, two objects on the DMA wavefronts "
               "(manual double buffering), LOAD_CACHE_STREAMING + STORE_LDS, 64 bytes per thread, two workgroups per compute unit")
        del s_src
    del pool

    # ---- config 3: indirect gather, row-sum consumer: the 512 MiB table of the configuration, and a 4 GiB table ----
    for name, recs, note, bound in (
            ("gather", 4 * 1024 * 1024, "CudaDMAIndirect 32 x 128 B records per tile from the configuration's 512 MiB table (4 Mi records, "
             "each read 8 times over per launch: most reads are served by L2 and the 256 MB Infinity Cache), two objects per DMA "
             "group with the index words requested one transfer ahead, three workgroups per compute unit, row-sum consumer",
             "infinity cache + hbm"),
            ("gather_hbm", 32 * 1024 * 1024, "the same kernel and index count on a 4 GiB table (32 Mi records, each read once on "
             "average; sixteen times the Infinity Cache), four workgroups per compute unit, row-sum consumer", "hbm")):
        if not want(name):
            continue
        table, idx, sums = inputs.pop(name)
        ms, _ = time_launches(lambda: wl.gather_rowsum(table, idx, sums, 0), steps, warmup, SETTLE_MS)
        report(patterns, name, ms, n_idx * 4 + n_idx * 128 + sums.numel() * 4, note, bound=bound)
        if want("yardsticks"):
            best_shape(lambda wg: (lambda: wl.probe_pattern("gather_xor", table, idx, sums, int(cus * wg))), (3, 4, 6), n_idx * 132 + sums.numel() * 4,
                       name + "_reads_alone", "the same index list and table read straight into registers (no LDS, no DMA object, xor instead of "
                       "the sum), 128 B written per 32 records; best of {tried} launch shapes: {best} workgroups per compute unit")
        del table, idx, sums

    # ---- the opposite direction (LDS -> global): scatter of 4 Mi records by a permutation ----
    if want("scatter"):
        recs = 4 * 1024 * 1024
        records, perm, table = inputs.pop("scatter")
        ms, _ = time_launches(lambda: wl.scatter_copy(records, perm, table, 0), steps, warmup, SETTLE_MS)
        report(patterns, "scatter", ms, recs * 4 + 2 * recs * 128,
               "CudaDMAIndirect<false> LDS -> global: 4 Mi records of 128 B placed by a permutation, 32 records per tile")
        if want("yardsticks"):
            best_shape(lambda wg: (lambda: wl.probe_pattern("scatter", records, perm, table, int(cus * wg))), (1, 2, 4), recs * 260,
                       "scatter_writes_alone", "the same records placed by the same permutation straight from registers (no LDS, no DMA "
                       "object); best of {tried} launch shapes: {best} workgroups per compute unit")
        del records, perm, table

    # ---- config 4: halo stencil ----
    if want("halo") or want("halo_handshake") or want("halo_wide_tiles"):
        g = 512
        grid_in, grid_out = inputs.pop("halo")
        if want("halo"):
            ms, _ = time_launches(lambda: wl.halo_stencil(grid_in, grid_out, 0), steps, warmup, SETTLE_MS)
            report(patterns, "halo", ms, 2 * g ** 3 * 4, "CudaDMAHalo radius-4 ring of 32x32 tiles, 25-point stencil on a 512^3 f32 grid "
                   "(ring landed without handshake, one s_barrier per plane)")
        if want("halo_handshake"):
            ms, _ = time_launches(lambda: wl.halo_stencil(grid_in, grid_out, 1), steps, warmup, SETTLE_MS)
            report(patterns, "halo_handshake", ms, 2 * g ** 3 * 4, "same kernel with the empty/full handshake on the LDS planes next to the s_barrier "
                   "(the split wait peek_dma_finish + wait_for_dma_finish(seen) keeps the poll off the critical path; the remaining cost is "
                   "the two LDS words per plane)")
            if "halo" in patterns:
                patterns["halo_handshake"]["time_vs_halo"] = round(ms / patterns["halo"]["ms"], 4)
        if want("halo_wide_tiles"):
            ms, _ = time_launches(lambda: wl.halo_stencil(grid_in, grid_out, wl.HALO_WIDE_TILES_VARIANT), steps, warmup, SETTLE_MS)
            report(patterns, "halo_wide_tiles", ms, 2 * g ** 3 * 4, "the kernel of the halo row with tiles of 64x16 cells (rows of 256 B in memory) "
                   "instead of the 32x32 tiles the configuration names")
        del grid_in, grid_out

    # ---- config 5: bf16 GEMM fed by CudaDMAStrided (MFMA-bound, reported in TFLOP/s); inputs normal(0,1) from seeds 1005 / 2005 ----
    gemm = None
    if want("gemm") or want("gemm_warp_specialised"):
        dim = 4096
        ga, gb, gc = inputs.pop("gemm")
        flops = 2.0 * dim ** 3
        mfma_busy = lambda name: (counters.get("patterns", {}).get(name) or {}).get("mfma_busy")

        def gemm_row(variant, name, note):
            ms, _ = time_launches(lambda: wl.gemm_bf16(ga, gb, gc, variant), max(steps, 50), warmup, SETTLE_MS)
            log(f"{name:24s} {ms:9.4f} ms  {flops / ms / 1e9:8.1f} TFLOP/s  {100 * flops / ms / 1e9 / MFMA_PEAK_TFLOPS:5.1f}% of 2.5 PFLOP/s")
            return {"TFLOP/s": round(flops / ms / 1e9, 1), "frac_of_mfma_peak": round(flops / ms / 1e9 / MFMA_PEAK_TFLOPS, 4),
                    "ms": round(ms, 4), "flop": flops, "kernel": PATTERN_KERNELS[name],
                    "mfma_busy_from_counters": mfma_busy(name), "workload": note}
        gemm = gemm_row(0, "gemm",
                        "C = A*B, bf16 4096^3 (A, B normal(0,1) from seeds 1005 / 2005), fp32 accumulate, 256x256 workgroup tile: B in four "
                        "stages of K=32, A in three buffers of K=64, brought into swizzled LDS by CudaDMAStrided::issue_direct_part "
                        "(global_load_lds) from the same four wavefronts that multiply (v_mfma_f32_32x32x16_bf16, 128x128 per "
                        "wavefront), one load between every four matrix instructions")
        gemm["note"] = ("config 5 names the warp-specialised kernel: it is reported under warp_specialised; the figures at "
                        "this level are the form of the same objects that is not warp-specialised")
        gemm["warp_specialised"] = gemm_row(wl.GEMM_WARP_SPECIALISED_VARIANT, "gemm_warp_specialised",
                                            "the same problem with DMA wavefronts feeding compute wavefronts through the handshake")
        if want("yardsticks") or want("vendor_gemm"):
            # the vendor library's GEMM (torch.matmul = hipBLASLt) on the same operands: the practical yardstick beside the peak
            ms, _ = time_launches(lambda: torch.matmul(ga, gb), max(steps, 50), warmup, SETTLE_MS)
            log(f"{'vendor_gemm':24s} {ms:9.4f} ms  {flops / ms / 1e9:8.1f} TFLOP/s  (torch.matmul, bf16 result)")
            gemm["vendor_library"] = {"TFLOP/s": round(flops / ms / 1e9, 1), "ms": round(ms, 4),
                                      "what": "torch.matmul (hipBLASLt) on the same bf16 operands, bf16 result"}
        del ga, gb, gc

    value = patterns["strided"]["GB/s"]
    copies = [yardsticks[k]["GB/s"] for k in ("plain_copy", "vendor_copy", "copy_best_shape") if k in yardsticks]
    ceiling = max(copies) if copies else None
    # every pattern against the yardstick of its own shape, measured in this run on the same buffers
    halo_traffic = None
    t_halo = traffic("halo")
    if t_halo:
        halo_traffic = t_halo / (2 * 512 ** 3 * 4)
    priced = {"strided": ("copy_best_shape", 1.0), "strided_settled": ("copy_best_shape", 1.0), "strided_even_split": ("copy_best_shape", 1.0),
              "strided_two_lds_tiles": ("copy_best_shape", 1.0),
              "strided_double_buffered_lds": ("copy_best_shape", 1.0), "sequential": ("copy_best_shape_64MiB", 1.0),
              "sequential_hbm": ("copy_best_shape", 1.0), "sequential_read_probe": ("read_only", 1.0),
              "gather": ("gather_reads_alone", 1.0), "gather_hbm": ("gather_hbm_reads_alone", 1.0), "scatter": ("scatter_writes_alone", 1.0),
              "halo": ("copy_best_shape", halo_traffic), "halo_handshake": ("copy_best_shape", halo_traffic),
              "halo_wide_tiles": ("copy_best_shape", halo_traffic)}
    for name, (stick, factor) in priced.items():
        if name in patterns and stick in yardsticks and factor:
            c = yardsticks[stick]["GB/s"] / factor
            patterns[name]["ceiling"] = round(c, 1)
            patterns[name]["frac_of_ceiling"] = round(patterns[name]["GB/s"] / c, 4)
            patterns[name]["ceiling_kind"] = f"yardsticks.{stick} of this run" + (
                "" if factor == 1.0 else f" divided by {factor:.3f}: the kernel's measured HBM traffic per algorithmic byte (ghost cells and padding)")
    roofline = {"bound": "hbm", "achieved": value, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(value / HBM_PEAK_GBS, 4), "traffic": traffic("strided"),
                "kernel": PATTERN_KERNELS["strided"], "kernel_ms": round(strided_ms, 4),
                "algorithmic_bytes_per_launch": strided_bytes,
                "ceiling": ceiling, "frac_of_ceiling": round(value / ceiling, 4) if ceiling else None,
                "ceiling_kind": "best read + write yardstick of this run on the same buffers (plain copy, hipMemcpyDtoDAsync, "
                                "copy at its best launch shape)",
                "counters_collected_at": counters.get("collected_at_commit")}
    if "read_only" in yardsticks and "write_only" in yardsticks:
        r, w = yardsticks["read_only"]["GB/s"], yardsticks["write_only"]["GB/s"]
        roofline["read_then_write_bound"] = round(2.0 / (1.0 / r + 1.0 / w), 1)     # 1 GiB read alone, then 1 GiB written alone
    result = {
        "metric": "achieved HBM GB/s (% of MI355X peak) per DMA pattern: seq/strided/gather/halo",
        "value": value,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(strided_wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "CudaDMAStrided 2D tile extraction: 16384x16384 f32, 64 rows x 256 B tiles at 65536 B stride, "
                               "double-buffered as one tile in LDS plus the next in the DMA wavefronts' registers (the forms with "
                               "two LDS tiles are patterns.strided_double_buffered_lds, one object, and patterns.strided_two_lds_tiles, "
                               "two objects), transposed to output (benchmark config 2 of 5)",
                   "tile_rows": 64, "tile_row_bytes": 256, "src_stride_bytes": 65536,
                   "workgroup": "192 DMA + 64 compute threads", "workgroups": "one per compute unit"},
        "roofline": roofline,
        "patterns": patterns,
        "yardsticks": yardsticks,
    }
    if gemm is not None:
        result["gemm"] = gemm
    bits, waves = cd.device_status(clear=True)
    result["handshake_waits_given_up"] = waves
    if bits or waves:
        sys.exit(f"bench.py: {waves} wavefront(s) gave up a handshake wait during the run: the figures are void")
    if not args.no_cpu_baseline:
        log("timing the host-core baselines (oracle, OpenMP) ...")
        result["cpu_baseline"], result["cpu_baseline_patterns"] = cpu_baselines()
        log(f"cpu baseline: {result['cpu_baseline']}")
        for name, row in result["cpu_baseline_patterns"].items():
            rate = f"{row['GB/s']:8.2f} GB/s" if "GB/s" in row else f"{row['TFLOP/s']:8.4f} TFLOP/s"
            log(f"  cpu {name:14s} {rate}   {row['sample']}")
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
