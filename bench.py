#!/usr/bin/env python3
"""Benchmark of the hipDMA transfer patterns on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one launch of the CudaDMAStrided tile-transpose kernel over the whole
16384 x 16384 float32 matrix (benchmark config 2, the configuration the metric is
quoted on); inputs are resident in HBM before the timed region.  The kernel is the
warp-specialised one with one LDS tile (the next tile waits in the DMA wavefronts'
registers), one workgroup per compute unit, streaming loads and stores; the kernel with two LDS tiles and two
objects, which needs four workgroups per compute unit, is reported beside it.  The other three
HBM-bound patterns (sequential copy, indirect gather, halo stencil), the scatter in
the opposite direction and a plain copy kernel are timed the same way and reported
under "patterns".  One JSON line goes to stdout; progress goes to stderr.
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
SETTLE_MS = 30.0                # wall time of untimed warm-up for the secondary patterns

# HBM bytes per launch of the headline kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE,
# scaled by what the same counters read for the plain copy kernel (see profiles/).
# profiles/bench_all_patterns_mi355x.md: FETCH_SIZE 524328 KiB x 1.99996 + WRITE_SIZE 1048598 KiB x 1.00000.
MEASURED_TRAFFIC_BYTES = {"strided": 2147566719}
# Matrix-core occupancy of the two GEMM kernels from rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CU_CYCLES
# (busy cycles / 4 SIMDs / busy cycles per compute unit), same file.
MEASURED_MFMA_BUSY = {"gemm": 0.739, "gemm_warp_specialised": 0.586}
STRIDED_VARIANT = 1             # cudadma_strided_transpose variant timed as the headline


def log(msg):
    print(msg, file=sys.stderr, flush=True)


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


def _median_time(fn, budget_s, min_reps=5, max_reps=400):
    fn()                                             # warm-up + first touch of the output
    times = []
    t_all = time.perf_counter()
    while len(times) < min_reps or (len(times) < max_reps and time.perf_counter() - t_all < budget_s):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return sorted(times)[len(times) // 2], len(times)


def cpu_baselines(budget_s=16.0):
    """The oracle's OpenMP implementation of each pattern on this machine's host cores, each on a
    bounded sample of its workload; bytes counted as for the GPU figures.  Returns the headline
    object (strided transpose) and a per-pattern dictionary."""
    import numpy as np
    from tests import oracle_lib as ol
    from tests.oracle_lib import ptr
    O = ol.load()
    cores = O.oracle_num_threads()
    per = budget_s / 5
    out = {}

    n = 8192                                         # a quarter of the matrix: 512 MiB of traffic per repetition
    a = ol.uniform(n * n, 1002).reshape(n, n)        # parallel first touch
    t = np.empty_like(a)
    med, reps = _median_time(lambda: O.oracle_transpose(ptr(a), ptr(t), n), per)
    out["strided"] = {"GB/s": round(2.0 * n * n * 4 / med / 1e9, 2),
                      "sample": f"oracle_transpose (256x256 tiles, 16x16 blocks through a local buffer) of an {n}x{n} float32 sample, median of {reps}"}
    del a, t

    m = 64 * 1024 * 1024 // 4                        # the whole config: 64 MiB
    src = ol.uniform(m, 1001)
    dst = np.empty_like(src)
    med, reps = _median_time(lambda: O.oracle_copy(ptr(src), ptr(dst), m), per)
    out["sequential"] = {"GB/s": round(2.0 * m * 4 / med / 1e9, 2),
                         "sample": f"oracle_copy of the full 64 MiB buffer (8 MiB per thread at 16 threads: resident in the host caches), median of {reps}"}
    del src, dst

    recs, n_idx = 4 * 1024 * 1024, 4 * 1024 * 1024   # full table, one eighth of the index list
    table = ol.uniform(recs * 32, 1003)
    idx = ol.indices(n_idx, recs, 1003)
    sums = np.empty(n_idx // 32 * 32, dtype=np.float32)
    med, reps = _median_time(lambda: O.oracle_gather_rowsum(ptr(table), ptr(idx), ptr(sums), n_idx, 32, 32), per)
    out["gather"] = {"GB/s": round((n_idx * 132 + sums.size * 4) / med / 1e9, 2),
                     "sample": f"oracle_gather_rowsum over the full 512 MiB table with {n_idx} indices, median of {reps}"}
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

    g, p = 256, 4                                    # one eighth of the grid
    grid = ol.uniform((g + 2 * p) ** 3, 1004)
    res = np.empty(g ** 3, dtype=np.float32)
    med, reps = _median_time(lambda: O.oracle_stencil25(ptr(grid), ptr(res), g, g, g, p), per)
    out["halo"] = {"GB/s": round(2.0 * g ** 3 * 4 / med / 1e9, 2),
                   "sample": f"oracle_stencil25 on a {g}^3 float32 sample, median of {reps}"}

    head = {"value": out["strided"]["GB/s"], "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "OpenMP " + out["strided"]["sample"]}
    return head, out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-core baseline leg")
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
    patterns = {}

    def report(name, ms, nbytes, note):
        gbs = nbytes / ms / 1e6
        patterns[name] = {"GB/s": round(gbs, 1), "frac_of_peak": round(gbs / HBM_PEAK_GBS, 4),
                          "ms": round(ms, 4), "algorithmic_bytes": nbytes, "workload": note}
        log(f"{name:12s} {ms:9.4f} ms  {gbs:8.1f} GB/s  {100 * gbs / HBM_PEAK_GBS:5.1f}% of peak   {note}")

    # ---- config 2: strided tile transpose (headline) ----
    n = 16384
    src = wl.fill_uniform(torch.empty(n * n, dtype=torch.float32, device=dev), 1002).view(n, n)
    dst = torch.empty_like(src)
    strided_ms, strided_wall_ms = time_launches(lambda: wl.strided_transpose(src, dst, STRIDED_VARIANT), steps, warmup)
    strided_bytes = 2 * n * n * 4
    report("strided", strided_ms, strided_bytes, "CudaDMAStrided 64x256B tiles of a 16384^2 f32 matrix, transposed out: one LDS tile, "
           "the next tile in the DMA wavefronts' registers, one workgroup per compute unit")
    ms, _ = time_launches(lambda: wl.strided_transpose(src, dst, 0), steps, warmup, SETTLE_MS)
    report("strided_two_lds_tiles", ms, strided_bytes, "the same transposition with two LDS tiles and two CudaDMAStrided objects "
           "(manual double buffering), four workgroups per compute unit")
    # yardstick on the same buffers: plain dwordx4 copy
    copy_ms, _ = time_launches(lambda: wl.plain_copy(src, dst), steps, warmup, SETTLE_MS)
    report("plain_copy", copy_ms, strided_bytes, "grid-stride dwordx4 copy of 1 GiB, no LDS, no DMA object")
    # two more yardsticks on the same buffers: the copy at its best launch shape, and the blocks of the
    # transposition moved through registers to their transposed position (no LDS, contents not transposed)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    flat_src, flat_dst = src.view(-1), dst.view(-1)
    ms, _ = time_launches(lambda: wl.probe_memory("copy_nontemporal", flat_src, flat_dst, 4 * cus), steps, warmup, SETTLE_MS)
    report("copy_best_shape", ms, strided_bytes, "the same copy with non-temporal stores at 4 workgroups per compute unit, its best launch shape")
    ms, _ = time_launches(lambda: wl.probe_memory("blocks_swapped", flat_src, flat_dst, 8 * cus), steps, warmup, SETTLE_MS)
    report("blocks_swapped", ms, strided_bytes, "64 x 256 B blocks through registers to the transposed block position: the placement cost of config 2 without LDS")
    del src, dst, flat_src, flat_dst

    # ---- config 1: sequential copy, 64 MiB in 16 KiB tiles ----
    m = 64 * 1024 * 1024 // 4
    s_src = wl.fill_uniform(torch.empty(m, dtype=torch.float32, device=dev), 1001)
    s_dst = torch.empty_like(s_src)
    ms, _ = time_launches(lambda: wl.sequential_copy(s_src, s_dst, 0), max(steps, 50), warmup, SETTLE_MS)
    report("sequential", ms, 2 * m * 4, "CudaDMASequential 16 KiB tiles of a 64 MiB f32 buffer (fits the 256 MB Infinity Cache)")
    del s_src, s_dst

    # ---- config 3: indirect gather, row-sum consumer ----
    recs, n_idx = 4 * 1024 * 1024, 32 * 1024 * 1024
    table = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, dtype=torch.float32, device=dev), 1003)
    idx = wl.fill_indices(torch.empty(n_idx, dtype=torch.int32, device=dev), recs, 1003)
    sums = torch.empty(n_idx // wl.RECS_PER_TILE * wl.REC_FLOATS, dtype=torch.float32, device=dev)
    ms, _ = time_launches(lambda: wl.gather_rowsum(table, idx, sums, 0), steps, warmup, SETTLE_MS)
    report("gather", ms, n_idx * 4 + n_idx * 128 + sums.numel() * 4,
           "CudaDMAIndirect 32 x 128 B records per tile from a 512 MiB table, row-sum consumer")
    del table, idx, sums

    # ---- the opposite direction (LDS -> global): scatter of 4 Mi records by a permutation ----
    records = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, dtype=torch.float32, device=dev), 1006)
    perm = wl.fill_permutation(torch.empty(recs, dtype=torch.int32, device=dev), 1006)
    table = torch.empty(recs * wl.REC_FLOATS, dtype=torch.float32, device=dev)
    ms, _ = time_launches(lambda: wl.scatter_copy(records, perm, table, 0), steps, warmup, SETTLE_MS)
    report("scatter", ms, recs * 4 + 2 * recs * 128,
           "CudaDMAIndirect<false> LDS -> global: 4 Mi records of 128 B placed by a permutation, 32 records per tile")
    del records, perm, table

    # ---- config 4: halo stencil ----
    g = 512
    p = 2 * wl.STENCIL_RADIUS
    grid_in = wl.fill_uniform(torch.empty((g + p) ** 3, dtype=torch.float32, device=dev), 1004).view(g + p, g + p, g + p)
    grid_out = torch.empty((g, g, g), dtype=torch.float32, device=dev)
    ms, _ = time_launches(lambda: wl.halo_stencil(grid_in, grid_out, 0), steps, warmup, SETTLE_MS)
    report("halo", ms, 2 * g ** 3 * 4, "CudaDMAHalo radius-4 ring of 32x32 tiles, 25-point stencil on a 512^3 f32 grid "
           "(ring landed without handshake, one s_barrier per plane)")
    ms, _ = time_launches(lambda: wl.halo_stencil(grid_in, grid_out, 1), steps, warmup, SETTLE_MS)
    report("halo_handshake", ms, 2 * g ** 3 * 4, "same kernel with the empty/full handshake on the LDS planes next to the s_barrier")
    del grid_in, grid_out

    # ---- config 5: warp-specialised bf16 GEMM (MFMA-bound, reported in TFLOP/s) ----
    dim = 4096
    ga = torch.randn((dim, dim), device=dev, dtype=torch.float32).to(torch.bfloat16)
    gb = torch.randn((dim, dim), device=dev, dtype=torch.float32).to(torch.bfloat16)
    gc = torch.empty((dim, dim), device=dev, dtype=torch.float32)
    ms, _ = time_launches(lambda: wl.gemm_bf16(ga, gb, gc), max(steps, 50), warmup, SETTLE_MS)
    flops = 2.0 * dim ** 3
    gemm = {"TFLOP/s": round(flops / ms / 1e9, 1), "frac_of_mfma_peak": round(flops / ms / 1e9 / 2500.0, 4),
            "ms": round(ms, 4), "flop": flops,
            "workload": "C = A*B, bf16 4096^3, fp32 accumulate, 256x256 workgroup tile: B in four stages of K=32, A in "
                        "three buffers of K=64, brought into swizzled LDS by CudaDMAStrided::issue_direct_part "
                        "(global_load_lds) from the same four wavefronts that multiply (v_mfma_f32_32x32x16_bf16, "
                        "128x128 per wavefront), one load between every four matrix instructions"}
    ms_ws, _ = time_launches(lambda: wl.gemm_bf16(ga, gb, gc, 7), max(steps, 50), warmup, SETTLE_MS)
    gemm["mfma_busy_from_counters"] = MEASURED_MFMA_BUSY["gemm"]
    gemm["note"] = ("config 5 names the warp-specialised kernel: it is reported under warp_specialised; the figures at "
                    "this level are the form of the same objects that is not warp-specialised, the faster one")
    gemm["warp_specialised"] = {"TFLOP/s": round(flops / ms_ws / 1e9, 1),
                                "frac_of_mfma_peak": round(flops / ms_ws / 1e9 / 2500.0, 4), "ms": round(ms_ws, 4),
                                "mfma_busy_from_counters": MEASURED_MFMA_BUSY["gemm_warp_specialised"],
                                "workload": "the same tile with four DMA wavefronts feeding eight compute wavefronts "
                                            "(128x64 per wavefront), variant 7"}
    log(f"gemm         {ms:9.4f} ms  {gemm['TFLOP/s']:8.1f} TFLOP/s  {100 * gemm['frac_of_mfma_peak']:5.1f}% of 2.5 PFLOP/s")
    log(f"gemm_ws      {ms_ws:9.4f} ms  {gemm['warp_specialised']['TFLOP/s']:8.1f} TFLOP/s  (warp-specialised, variant 7)")
    del ga, gb, gc

    value = patterns["strided"]["GB/s"]
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
                               "one tile in LDS and the next in the DMA wavefronts' registers, transposed to output "
                               "(benchmark config 2 of 5)",
                   "tile_rows": 64, "tile_row_bytes": 256, "src_stride_bytes": 65536,
                   "workgroup": "128 DMA + 128 compute threads", "workgroups": "one per compute unit"},
        "roofline": {"bound": "hbm", "achieved": value, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(value / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES["strided"],
                     "kernel": "transpose_single<true, true>", "kernel_ms": round(strided_ms, 4),
                     "algorithmic_bytes_per_launch": strided_bytes},
        "patterns": patterns,
        "gemm": gemm,
    }
    if not args.no_cpu_baseline:
        log("timing the host-core baselines (oracle, OpenMP) ...")
        result["cpu_baseline"], result["cpu_baseline_patterns"] = cpu_baselines()
        log(f"cpu baseline: {result['cpu_baseline']}")
        for name, row in result["cpu_baseline_patterns"].items():
            log(f"  cpu {name:10s} {row['GB/s']:8.2f} GB/s   {row['sample']}")
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
