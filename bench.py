#!/usr/bin/env python3
"""Benchmark of the hipDMA transfer patterns on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME[,NAME...]] [--no-cpu-baseline]

A step is one launch of the CudaDMAStrided tile-transpose kernel over the whole 16384 x 16384 float32
matrix (benchmark config 2, the configuration the metric is quoted on); inputs are resident in HBM before
the timed region.  The other HBM-bound patterns (sequential copy, indirect gather, halo stencil), the scatter
in the opposite direction and the GEMM are timed the same way (HIP events on the launch stream) and reported
under "patterns" / "gemm".  The sequential copy and the gather are each reported twice: at the size the
configuration names (64 MiB buffer, 512 MiB table: both working sets are helped by the 256 MB Infinity Cache)
and at a size that is not (1 GiB buffer, 4 GiB table).  "yardsticks" holds what read-only, write-only and
copy-shaped streams and the vendor's own device-to-device copy reach on the same 1 GiB buffers in the same
run; roofline.ceiling is the best read + write yardstick of the run.  Counter-derived fields (HBM traffic per
launch, matrix-core occupancy) come from profiles/counters.json, which `python -m cudadma_amd.profile_summary`
writes from rocprofv3 output.  One JSON line goes to stdout; progress goes to stderr.
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
    "strided": "transpose_split<3, 1, 1>",
    "strided_even_split": "transpose_single<true, true>",
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

    def report(table, name, ms, nbytes, note, bound="hbm"):
        gbs = nbytes / ms / 1e6
        row = {"GB/s": round(gbs, 1), "frac_of_peak": round(gbs / HBM_PEAK_GBS, 4), "ms": round(ms, 4),
               "algorithmic_bytes": nbytes, "bound": bound, "workload": note}
        if table is patterns:
            row["kernel"] = PATTERN_KERNELS.get(name)
            row["traffic_bytes_from_counters"] = traffic(name)
        table[name] = row
        log(f"{name:24s} {ms:9.4f} ms  {gbs:8.1f} GB/s  {100 * gbs / HBM_PEAK_GBS:5.1f}% of peak   {note}")

    # ---- config 2: strided tile transpose (headline) ----
    # One allocation holds the source and, exactly 1 GiB behind it, the destination of every 1 GiB + 1 GiB stream of
    # this run: the rate of a linear copy depends on the distance between its two buffers (0.350 to 0.440 ms for the
    # same kernel as the distance varies modulo 64 MiB; the transposition does not care), and two separate
    # allocations land wherever the allocator, or a profiler loaded into the process, leaves room.
    n = 16384
    pool = torch.empty(2 * n * n, dtype=torch.float32, device=dev)
    src = wl.fill_uniform(pool[:n * n], 1002).view(n, n)
    dst = pool[n * n:].view(n, n)
    strided_ms, strided_wall_ms = time_launches(lambda: wl.strided_transpose(src, dst, STRIDED_VARIANT), steps, warmup)
    strided_bytes = 2 * n * n * 4
    report(patterns, "strided", strided_ms, strided_bytes,
           "CudaDMAStrided 64x256B tiles of a 16384^2 f32 matrix, transposed out: one LDS tile, the next tile in the DMA "
           "wavefronts' registers (the double buffer is LDS + registers), one workgroup of three DMA wavefronts and one "
           "compute wavefront per compute unit")
    if want("strided_even_split"):
        ms, _ = time_launches(lambda: wl.strided_transpose(src, dst, 1), steps, warmup, SETTLE_MS)
        report(patterns, "strided_even_split", ms, strided_bytes, "the same kernel shape with two DMA and two compute wavefronts (128 + 128 threads)")
    if want("strided_two_lds_tiles"):
        ms, _ = time_launches(lambda: wl.strided_transpose(src, dst, wl.TRANSPOSE_TWO_LDS_TILES_VARIANT), steps, warmup, SETTLE_MS)
        report(patterns, "strided_two_lds_tiles", ms, strided_bytes,
               "the same transposition with two LDS tiles and two CudaDMAStrided objects (manual double buffering in LDS)")
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

        def best_shape(modes, s_, d_, shapes, nbytes, label):
            best = None
            for mode in modes:
                for wg in shapes:
                    ms, _ = time_launches(lambda: wl.probe_memory(mode, s_, d_, int(cus * wg)), max(10, steps // 2), 5, 10.0)
                    if best is None or ms < best[0]:
                        best = (ms, wg, mode)
            report(yardsticks, label, best[0], nbytes,
                   f"{best[2]} stream over 1 GiB, grid-stride dwordx4, best of {len(modes) * len(shapes)} (cache hint, launch shape) "
                   f"pairs: {best[1]} workgroups per compute unit")
        best_shape(("read", "read_nontemporal"), flat_src, None, (1, 1.5, 2, 3, 4), strided_bytes // 2, "read_only")
        best_shape(("write", "write_nontemporal"), None, flat_dst, (0.5, 1, 2, 4), strided_bytes // 2, "write_only")
        best_shape(("copy", "copy_nontemporal"), flat_src, flat_dst, (1, 2, 4, 8), strided_bytes, "copy_best_shape")
    del src, dst, flat_src, flat_dst

    # ---- config 1: sequential copy in 16 KiB tiles: the 64 MiB of the configuration, and 1 GiB ----
    if want("sequential"):
        m = 64 * 1024 * 1024 // 4
        s_src = wl.fill_uniform(torch.empty(m, dtype=torch.float32, device=dev), 1001)
        s_dst = torch.empty_like(s_src)
        ms, _ = time_launches(lambda: wl.sequential_copy(s_src, s_dst, 0), max(steps, 50), warmup, SETTLE_MS)
        report(patterns, "sequential", ms, 2 * m * 4, "CudaDMASequential 16 KiB tiles of the configuration's 64 MiB f32 buffer: the "
               "128 MiB working set stays in the 256 MB Infinity Cache from launch to launch, so this is a cache-assisted rate, "
               "not an HBM rate", bound="infinity cache + hbm")
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
    del pool

    # ---- config 3: indirect gather, row-sum consumer: the 512 MiB table of the configuration, and a 4 GiB table ----
    n_idx = 32 * 1024 * 1024
    for name, recs, note, bound in (
            ("gather", 4 * 1024 * 1024, "CudaDMAIndirect 32 x 128 B records per tile from the configuration's 512 MiB table (4 Mi records, "
             "each read 8 times over per launch: most reads are served by L2 and the 256 MB Infinity Cache), two objects per DMA "
             "group with the index words requested one transfer ahead, three workgroups per compute unit, row-sum consumer",
             "infinity cache + hbm"),
            ("gather_hbm", 32 * 1024 * 1024, "the same kernel and index count on a 4 GiB table (32 Mi records, each read once on "
             "average; sixteen times the Infinity Cache), four workgroups per compute unit, row-sum consumer", "hbm")):
        if not want(name):
            continue
        table = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, dtype=torch.float32, device=dev), 1003)
        idx = wl.fill_indices(torch.empty(n_idx, dtype=torch.int32, device=dev), recs, 1003)
        sums = torch.empty(n_idx // wl.RECS_PER_TILE * wl.REC_FLOATS, dtype=torch.float32, device=dev)
        ms, _ = time_launches(lambda: wl.gather_rowsum(table, idx, sums, 0), steps, warmup, SETTLE_MS)
        report(patterns, name, ms, n_idx * 4 + n_idx * 128 + sums.numel() * 4, note, bound=bound)
        del table, idx, sums

    # ---- the opposite direction (LDS -> global): scatter of 4 Mi records by a permutation ----
    if want("scatter"):
        recs = 4 * 1024 * 1024
        records = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, dtype=torch.float32, device=dev), 1006)
        perm = wl.fill_permutation(torch.empty(recs, dtype=torch.int32, device=dev), 1006)
        table = torch.empty(recs * wl.REC_FLOATS, dtype=torch.float32, device=dev)
        ms, _ = time_launches(lambda: wl.scatter_copy(records, perm, table, 0), steps, warmup, SETTLE_MS)
        report(patterns, "scatter", ms, recs * 4 + 2 * recs * 128,
               "CudaDMAIndirect<false> LDS -> global: 4 Mi records of 128 B placed by a permutation, 32 records per tile")
        del records, perm, table

    # ---- config 4: halo stencil ----
    if want("halo") or want("halo_handshake") or want("halo_wide_tiles"):
        g = 512
        p = 2 * wl.STENCIL_RADIUS
        grid_in = wl.fill_uniform(torch.empty((g + p) ** 3, dtype=torch.float32, device=dev), 1004).view(g + p, g + p, g + p)
        grid_out = torch.empty((g, g, g), dtype=torch.float32, device=dev)
        if want("halo"):
            ms, _ = time_launches(lambda: wl.halo_stencil(grid_in, grid_out, 0), steps, warmup, SETTLE_MS)
            report(patterns, "halo", ms, 2 * g ** 3 * 4, "CudaDMAHalo radius-4 ring of 32x32 tiles, 25-point stencil on a 512^3 f32 grid "
                   "(ring landed without handshake, one s_barrier per plane)")
        if want("halo_handshake"):
            ms, _ = time_launches(lambda: wl.halo_stencil(grid_in, grid_out, 1), steps, warmup, SETTLE_MS)
            report(patterns, "halo_handshake", ms, 2 * g ** 3 * 4, "same kernel with the empty/full handshake on the LDS planes next to the s_barrier")
        if want("halo_wide_tiles"):
            ms, _ = time_launches(lambda: wl.halo_stencil(grid_in, grid_out, wl.HALO_WIDE_TILES_VARIANT), steps, warmup, SETTLE_MS)
            report(patterns, "halo_wide_tiles", ms, 2 * g ** 3 * 4, "the kernel of the halo row with tiles of 64x16 cells (rows of 256 B in memory) "
                   "instead of the 32x32 tiles the configuration names")
        del grid_in, grid_out

    # ---- config 5: bf16 GEMM fed by CudaDMAStrided (MFMA-bound, reported in TFLOP/s); inputs normal(0,1) from seeds 1005 / 2005 ----
    gemm = None
    if want("gemm") or want("gemm_warp_specialised"):
        dim = 4096
        ga = wl.fill_normal_bf16(torch.empty((dim, dim), device=dev, dtype=torch.bfloat16), 1005)
        gb = wl.fill_normal_bf16(torch.empty((dim, dim), device=dev, dtype=torch.bfloat16), 2005)
        gc = torch.empty((dim, dim), device=dev, dtype=torch.float32)
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
                               "double-buffered as one tile in LDS plus the next in the DMA wavefronts' registers (the form with "
                               "two LDS tiles is patterns.strided_two_lds_tiles), transposed to output (benchmark config 2 of 5)",
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
            log(f"  cpu {name:14s} {row['GB/s']:8.2f} GB/s   {row['sample']}")
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
