"""Parameter sweep over the benchmark workloads: every buffering variant x workgroups per
compute unit, timed with HIP events.  The counterpart of the reference's
src/perf/sequential/param_sweep.py:27-58, which rewrites params_directed.h and recompiles per
point; here the variants are compiled in and the occupancy is a run-time knob.

    python -m cudadma_amd.sweep [sequential] [strided] [gather] [gather_hbm] [scatter] [halo] [gemm] [yardsticks] [--wg 0,2,4,8] [--steps 20]
    python -m cudadma_amd.sweep saxpy sgemv stencil2d        # the reference's example programs, every variant
    python -m cudadma_amd.sweep perf_sequential --wg 2,8     # read-bandwidth probe: element size x DMA wavefronts x buffering
    python -m cudadma_amd.sweep transpose_split              # DMA : compute wavefronts x tiles ahead x workgroups per CU
    python -m cudadma_amd.sweep transpose_walk               # tile order x workgroup count, one-tile and two-tile kernels
    python -m cudadma_amd.sweep placement                    # 1 GiB copies against the distance between source and destination
    python -m cudadma_amd.sweep placement_fine               # the copy yardstick alone against 51 distances from 0 to 256 MiB
    python -m cudadma_amd.sweep pattern_yardsticks           # the patterns' own addresses without LDS or objects, next to the patterns
    python -m cudadma_amd.sweep gather_reach                 # the gather against the size of its table, 128 MiB to 16 GiB
    python -m cudadma_amd.sweep pattern_pitch                # the tile-shaped reads and writes alone, and the kernel, on matrices whose row pitch is not a power of two
    python -m cudadma_amd.sweep channel_hash                 # which address bits choose the memory channel: half of a 1 GiB buffer by the parity of 1-3 bits
    python -m cudadma_amd.sweep settle                       # the first 80 launches after an idle second, one by one, with the shader clock
    python -m cudadma_amd.sweep two_streams                  # a read-only kernel and a write-only kernel side by side against one copy kernel
    python -m cudadma_amd.sweep queue_depth --config NAME    # one launch shape of QUEUE_CONFIGS, a few launches: the process to put
                                                             # under rocprofv3 --pmc when asking what more work in flight costs
"""
import argparse
import sys

import torch

from . import examples as ex
from . import workloads as wl

PEAK_GBS = 8000.0

# Launch shapes that differ only in how much work a compute unit has in flight: (what to launch, knobs / workgroups per compute
# unit).  `python -m cudadma_amd.sweep queue_depth --config NAME` runs one of them on 2 x 1 GiB; cudadma_amd.profile_summary
# tabulates the counters of such runs.
QUEUE_CONFIGS = {
    "transpose_1wg_1tile": ("transpose", {"transpose_split": 311, "transpose_workgroups": 1}),
    "transpose_2wg_1tile": ("transpose", {"transpose_split": 311, "transpose_workgroups": 2}),
    "transpose_1wg_2tiles": ("transpose", {"transpose_split": 312, "transpose_workgroups": 1}),
    "transpose_2wg_2tiles": ("transpose", {"transpose_split": 312, "transpose_workgroups": 2}),
    "copy_2wg": ("copy_nontemporal", 2), "copy_4wg": ("copy_nontemporal", 4), "copy_8wg": ("copy_nontemporal", 8),
    "copy_16wg": ("copy_nontemporal", 16),
    "read_1.5wg": ("read_nontemporal", 1.5), "read_4wg": ("read_nontemporal", 4), "read_8wg": ("read_nontemporal", 8),
    "write_0.5wg": ("write", 0.5), "write_4wg": ("write", 4), "write_8wg": ("write", 8),
    # cached against non-temporal loads: the plain read stream, and the read-bandwidth probe on CudaDMASequential
    # (16 KiB elements, four DMA wavefronts, manual double buffering, two workgroups per compute unit)
    "read_cached_1.5wg": ("read", 1.5),
    "probe_cached": ("perf_sequential", "LOAD_CACHE_ALL"), "probe_streaming": ("perf_sequential", "LOAD_CACHE_STREAMING"),
    # the patterns' own addresses through bare loads or stores (cudadma_probe_pattern): (mode, piece bytes, workgroups per
    # compute unit, XCD grouping) -- the transposition's destination tiles written in pieces of 256 B (its own shape), 1 KiB and
    # 4 KiB, its source tiles read, the scatter's permutation written, the gather's index list read from a 4 GiB table
    "tile_write_256": ("pattern", ("tile_write", 256, 1, 0)), "tile_write_1024": ("pattern", ("tile_write", 1024, 0.5, 0)),
    "tile_write_4096_grouped": ("pattern", ("tile_write", 4096, 0.5, 1)), "tile_read_256": ("pattern", ("tile_read", 256, 1.5, 0)),
    "scatter_writes": ("pattern", ("scatter", 0, 1, 0)), "gather_hbm_reads": ("pattern", ("gather_xor", 0, 4, 0)),
    # the gather of 32 Mi random 128-byte records from a table of 512 MiB and of 4 GiB: bare loads (3 and 4 workgroups per
    # compute unit) and the reported CudaDMAIndirect kernel
    "gather_reads": ("pattern", ("gather_xor_small", 0, 3, 0)),
    "gather_reads_1GiB": ("pattern", ("gather_xor_8Mi", 0, 4, 0)), "gather_reads_2GiB": ("pattern", ("gather_xor_16Mi", 0, 4, 0)),
    "gather_reads_16GiB": ("pattern", ("gather_xor_128Mi", 0, 4, 0)),
    "gather_dma": ("pattern", ("gather_dma_small", 0, 0, 0)), "gather_hbm_dma": ("pattern", ("gather_dma", 0, 0, 0)),
}


def _time(fn, steps, warmup=3, settle_ms=30.0):
    """Average milliseconds per launch.  Warm-up runs for at least `warmup` launches and `settle_ms`
    of wall time: the first launches after an idle or allocation phase run up to 25 % slow."""
    import time
    t0 = time.perf_counter()
    done = 0
    while done < warmup or (time.perf_counter() - t0) * 1e3 < settle_ms:
        fn()
        done += 1
        if done % 8 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    a = torch.cuda.Event(enable_timing=True)
    b = torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / steps


def _row(name, variant, wg, ms, nbytes):
    gbs = nbytes / ms / 1e6
    print(f"{name:10s} variant {variant}  wg/cu {wg:2d}  {ms:9.4f} ms  {gbs:8.0f} GB/s  {100 * gbs / PEAK_GBS:5.1f}%", flush=True)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("workloads", nargs="*", default=["sequential", "strided", "gather", "halo", "gemm"])
    ap.add_argument("--wg", default="0,2,4,8", help="workgroups per compute unit to try (0 = each kernel's default)")
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--config", default="", help="queue_depth: name of the launch shape (see QUEUE_CONFIGS)")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        sys.exit("no GPU visible")
    dev = torch.device("cuda:0")
    wgs = [int(x) for x in args.wg.split(",")]
    for name in args.workloads:
        if name == "sequential":
            src = wl.fill_uniform(torch.empty(16 << 20, device=dev), 1001)
            dst = torch.empty_like(src)
            for v in wl.variants(wl.SEQUENTIAL):
                print(f"# sequential variant {v}: {wl.variant_name(wl.SEQUENTIAL, v)}")
                for wg in wgs:
                    wl.set_workgroups_per_cu(wg)
                    _row(name, v, wg, _time(lambda: wl.sequential_copy(src, dst, v), max(args.steps, 50)), 2 * src.numel() * 4)
        elif name == "strided":
            n = 16384
            src = wl.fill_uniform(torch.empty(n * n, device=dev), 1002).view(n, n)
            dst = torch.empty_like(src)
            for v in wl.variants(wl.STRIDED):
                print(f"# strided variant {v}: {wl.variant_name(wl.STRIDED, v)}")
                for wg in wgs:
                    wl.set_workgroups_per_cu(wg)
                    _row(name, v, wg, _time(lambda: wl.strided_transpose(src, dst, v), args.steps), 2 * n * n * 4)
        elif name in ("gather", "gather_hbm"):
            # the configuration's 512 MiB table, or one of 4 GiB (sixteen times the Infinity Cache)
            recs, n_idx = (4 << 20) if name == "gather" else (32 << 20), 32 << 20
            table = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, device=dev), 1003)
            idx = wl.fill_indices(torch.empty(n_idx, dtype=torch.int32, device=dev), recs, 1003)
            out = torch.empty(n_idx // wl.RECS_PER_TILE * wl.REC_FLOATS, device=dev)
            for v in wl.variants(wl.GATHER):
                print(f"# gather (row-sum) variant {v}: {wl.variant_name(wl.GATHER, v)}")
                for wg in wgs:
                    wl.set_workgroups_per_cu(wg)
                    _row(name, v, wg, _time(lambda: wl.gather_rowsum(table, idx, out, v), args.steps),
                         n_idx * 132 + out.numel() * 4)
        elif name == "yardsticks":
            # read-only, write-only and copy streams on 2 x 1 GiB per launch shape, and the vendor's copy
            n = 16384
            src = wl.fill_uniform(torch.empty(n * n, device=dev), 1002)
            dst = torch.empty_like(src)
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            shapes = (0.5, 1, 1.5, 2, 3, 4, 8, 16)
            print("# streaming yardsticks on 2 x 1 GiB; ms and GB/s of bytes read + written; columns: workgroups per CU " + " / ".join(map(str, shapes)))
            for mode, label in enumerate(wl.PROBE_MODES):
                cells = []
                for wg in (shapes if label != "vendor_copy" else (1,)):
                    s_, d_ = (None if label.startswith("write") else src), (None if label.startswith("read") else dst)
                    nbytes = wl.probe_memory(mode, s_, d_, int(cus * wg))
                    ms = _time(lambda: wl.probe_memory(mode, s_, d_, int(cus * wg)), args.steps, settle_ms=10.0)
                    cells.append(f"{ms:7.4f} ms {nbytes / ms / 1e6:6.0f}")
                print(f"{label:22s} " + "   ".join(cells), flush=True)
        elif name == "transpose_split":
            # the transposition of config 2 with every compiled (DMA wavefronts, compute wavefronts, tiles ahead)
            # split, at one, two and three workgroups per compute unit; each split is checked against torch first
            n = 16384
            src = wl.fill_uniform(torch.empty(n * n, device=dev), 1002).view(n, n)
            dst = torch.empty_like(src)
            ref = src.t().contiguous()
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            print("# DMA + compute wavefronts, tiles ahead: ms (% of 8 TB/s) at 1 / 2 / 3 workgroups per compute unit")
            for code in wl.transpose_splits():
                wl.set_tuning("transpose_split", code)
                dst.zero_()
                wl.strided_transpose(src, dst, wl.TRANSPOSE_SPLIT_VARIANT)
                exact = torch.equal(dst, ref)
                cells = []
                for wg in (1, 2, 3):
                    wl.set_tuning("transpose_workgroups", cus * wg)
                    ms = _time(lambda: wl.strided_transpose(src, dst, wl.TRANSPOSE_SPLIT_VARIANT), args.steps, settle_ms=15.0)
                    cells.append(f"{ms:.4f} ({2 * n * n * 4 / ms / 1e6 / PEAK_GBS * 100:4.1f}%)")
                wl.set_tuning("transpose_workgroups", 0)
                ahead = {3: "1.5 (3 halves)", 4: "1.25 (5 quarters)", 5: "1.5 (6 quarters)", 6: "1.75 (7 quarters)",
                         7: "0.75 (3 quarters)", 8: "1, requested on return,"}.get(code % 10, str(code % 10))
                print(f"{code // 100} + {code // 10 % 10}, {ahead} ahead:  " + "   ".join(cells) + ("" if exact else "   WRONG RESULT"),
                      flush=True)
            wl.set_tuning("transpose_split", 0)
            del ref
        elif name == "transpose_walk":
            # the order in which the tiles are taken (bands of `band` tile rows; a band as high as the matrix walks down
            # the columns, so every workgroup stays on its own 64 matrix rows) against the number of workgroups, for the
            # kernels with one tile per workgroup in flight (variants 0, 1) and with two (variants 11, 3, 5)
            n = 16384
            src = wl.fill_uniform(torch.empty(n * n, device=dev), 1002).view(n, n)
            dst = torch.empty_like(src)
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            counts = (cus // 2, cus * 3 // 4, cus - 8, cus, cus + 8, cus * 2, cus * 4)
            print("# variant, band: % of 8 TB/s with " + " / ".join(str(c) for c in counts) + " workgroups")
            for variant in (0, 1, wl.TRANSPOSE_TWO_LDS_TILES_VARIANT, 3, 5):
                for band in (256, 64, 16, 4, 1):
                    wl.set_tuning("transpose_band", band)
                    cells = []
                    for count in counts:
                        wl.set_tuning("transpose_workgroups", count)
                        ms = _time(lambda: wl.strided_transpose(src, dst, variant), args.steps, settle_ms=10.0)
                        cells.append(f"{2 * n * n * 4 / ms / 1e6 / PEAK_GBS * 100:4.1f}")
                    print(f"variant {variant:2d}  band {band:3d}:  " + "  ".join(cells), flush=True)
            wl.set_tuning("transpose_band", 0)
            wl.set_tuning("transpose_workgroups", 0)
        elif name == "placement":
            # linear copies of 1 GiB inside one allocation, against the distance from source to destination;
            # the transposition of the same bytes beside them
            m = (1 << 30) // 4
            pool = torch.empty(2 * m + (64 << 20) // 4, device=dev)
            src = wl.fill_uniform(pool[:m], 1001)
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            print("# destination - source = 1 GiB + offset: ms (% of 8 TB/s) of sequential variant 5 (tile-interleaved) / variant 6 "
                  "(contiguous runs) / copy_nontemporal yardstick at 4 workgroups per CU / transposition (headline variant)")
            for off in (0, 4096, 16384, 65536, 1 << 20, 2 << 20, 4 << 20, 8 << 20, 16 << 20, (16 << 20) + 4096, 24 << 20,
                        32 << 20, 48 << 20, 64 << 20):
                dst = pool[m + off // 4: 2 * m + off // 4]
                cells = []
                for fn in (lambda: wl.sequential_copy(src, dst, 5), lambda: wl.sequential_copy(src, dst, 6),
                           lambda: wl.probe_memory("copy_nontemporal", src, dst, cus * 4),
                           lambda: wl.strided_transpose(src.view(16384, 16384), dst.view(16384, 16384), 0)):
                    ms = _time(fn, args.steps, settle_ms=15.0)
                    cells.append(f"{ms:.4f} ({2 * m * 4 / ms / 1e6 / PEAK_GBS * 100:4.1f}%)")
                print(f"+{off:>9d} B:  " + "   ".join(cells), flush=True)
            del pool
        elif name == "placement_fine":
            m = (1 << 30) // 4
            pool = torch.empty(2 * m + (256 << 20) // 4, device=dev)
            src = wl.fill_uniform(pool[:m], 1001)
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            K, M = 1 << 10, 1 << 20
            offs = [0, 256, 512, 1 * K, 2 * K, 3 * K, 4 * K, 6 * K, 8 * K, 12 * K, 16 * K, 20 * K, 24 * K, 28 * K, 32 * K, 40 * K, 48 * K, 56 * K,
                    64 * K, 80 * K, 96 * K, 128 * K, 192 * K, 256 * K, 384 * K, 512 * K, 768 * K, 1 * M, 1536 * K, 2 * M, 3 * M, 4 * M, 5 * M, 6 * M,
                    8 * M, 10 * M, 12 * M, 14 * M, 16 * M, 20 * M, 24 * M, 28 * M, 32 * M, 40 * M, 48 * M, 56 * M, 64 * M, 96 * M, 128 * M, 192 * M,
                    256 * M]
            print("# copy_nontemporal yardstick, destination - source = 1 GiB + offset: % of 8 TB/s at 3 / 4 / 6 workgroups per compute unit")
            for off in offs:
                dst = pool[m + off // 4: 2 * m + off // 4]
                cells = []
                for wg in (3, 4, 6):
                    ms = _time(lambda: wl.probe_memory("copy_nontemporal", src, dst, cus * wg), args.steps, settle_ms=8.0)
                    cells.append(f"{2 * m * 4 / ms / 1e6 / PEAK_GBS * 100:5.1f}")
                print(f"+{off:>10d} B ({off / K:10.2f} KiB):  " + "  ".join(cells), flush=True)
            del pool
        elif name == "pattern_yardsticks":
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            pct = lambda nb, ms: f"{nb / ms / 1e6 / PEAK_GBS * 100:5.1f}"
            n_idx = 32 << 20
            for recs in (4 << 20, 32 << 20):
                table = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, device=dev), 1003)
                idx = wl.fill_indices(torch.empty(n_idx, dtype=torch.int32, device=dev), recs, 1003)
                out = torch.empty(n_idx // wl.RECS_PER_TILE * wl.REC_FLOATS, device=dev)
                shapes = (2, 3, 4, 6, 8)
                nb = n_idx * 132 + out.numel() * 4
                cells = [pct(nb, _time(lambda: wl.probe_pattern("gather_xor", table, idx, out, cus * wg), args.steps, settle_ms=10.0)) for wg in shapes]
                dma = pct(nb, _time(lambda: wl.gather_rowsum(table, idx, out, 0), args.steps, settle_ms=10.0))
                print(f"gather, table of {recs >> 20} Mi records: records read straight into registers " + " / ".join(cells) +
                      f" % of 8 TB/s at {shapes} workgroups per CU; cudadma_gather_rowsum {dma} %", flush=True)
                del table, idx, out
            recs = 4 << 20
            records = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, device=dev), 1006)
            perm = wl.fill_permutation(torch.empty(recs, dtype=torch.int32, device=dev), 1006)
            table = torch.empty(recs * wl.REC_FLOATS, device=dev)
            shapes = (1, 2, 3, 4, 6, 8)
            cells = [pct(recs * 260, _time(lambda: wl.probe_pattern("scatter", records, perm, table, cus * wg), args.steps, settle_ms=10.0)) for wg in shapes]
            dma = pct(recs * 260, _time(lambda: wl.scatter_copy(records, perm, table, 0), args.steps, settle_ms=10.0))
            print(f"scatter of {recs >> 20} Mi records: records written straight from registers " + " / ".join(cells) +
                  f" % at {shapes} workgroups per CU; cudadma_scatter_copy {dma} %", flush=True)
            del records, perm, table
            n = 16384
            pool = torch.empty(2 * n * n, device=dev)
            src = wl.fill_uniform(pool[:n * n], 1002).view(n, n)
            dst = pool[n * n:].view(n, n)
            sink = torch.empty(8 * cus * 4, device=dev)
            shapes = (0.5, 1, 1.5, 2, 3, 4)
            cells = [pct(n * n * 4, _time(lambda: wl.probe_pattern("tile_read", src, None, sink, int(cus * wg)), args.steps, settle_ms=10.0)) for wg in shapes]
            print("transposition, its source tiles read alone: " + " / ".join(cells) + f" % at {shapes} workgroups per CU", flush=True)
            for mode, shapes in (("tile_write", (0.5, 1, 1.5, 2, 3, 4)), ("tile_copy", (1, 2, 3, 4, 6, 8))):
                for xg in (0, 1):
                    wl.set_tuning("probe_xcd_group", xg)
                    for piece in (256, 512, 1024, 2048, 4096):
                        wl.set_tuning("probe_piece_bytes", piece)
                        nb = n * n * 4 * (2 if mode == "tile_copy" else 1)
                        s_ = src if mode == "tile_copy" else None
                        cells = [pct(nb, _time(lambda: wl.probe_pattern(mode, s_, None, dst, int(cus * wg)), args.steps, settle_ms=10.0)) for wg in shapes]
                        print(f"transposition, {mode} in pieces of {piece:4d} B, XCD grouping {xg}: " + " / ".join(cells) +
                              f" % at {shapes} workgroups per CU", flush=True)
            wl.set_tuning("probe_piece_bytes", 0)
            wl.set_tuning("probe_xcd_group", 0)
            ms = _time(lambda: wl.strided_transpose(src, dst, 0), args.steps, settle_ms=20.0)
            print(f"cudadma_strided_transpose variant 0: {pct(2 * n * n * 4, ms)} %", flush=True)
            del pool
        elif name == "gather_reach":
            # the gather of 32 Mi random 128-byte records against the size of the table they come from: where the rate leaves
            # the cache-assisted figure, and where address translation starts to miss (counters: queue_depth gather_*)
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            n_idx = 32 << 20
            out = torch.empty(n_idx // wl.RECS_PER_TILE * wl.REC_FLOATS, device=dev)
            nb = n_idx * 132 + out.numel() * 4
            for mib in (128, 256, 512, 768, 1024, 1536, 2048, 3072, 4096, 8192, 16384):
                recs = mib << 13
                table = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, device=dev), 1003)
                idx = wl.fill_indices(torch.empty(n_idx, dtype=torch.int32, device=dev), recs, 1003)
                bare = [nb / _time(lambda: wl.probe_pattern("gather_xor", table, idx, out, cus * wg), args.steps, settle_ms=10.0) / 1e6 / PEAK_GBS * 100
                        for wg in (3, 4)]
                dma = nb / _time(lambda: wl.gather_rowsum(table, idx, out, 0), args.steps, settle_ms=10.0) / 1e6 / PEAK_GBS * 100
                print(f"gather_reach  table {mib:6d} MiB: records read into registers {bare[0]:5.1f} / {bare[1]:5.1f} % at 3 / 4 workgroups per CU; "
                      f"cudadma_gather_rowsum {dma:5.1f} %", flush=True)
                del table, idx
        elif name == "pattern_pitch":
            # is the transposition's write side held back by the power-of-two row pitch (every row of a tile on the same
            # low address bits: the same cache channel and set)?  The tile-shaped reads and writes alone and the kernel,
            # on square matrices of other sizes
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            pct = lambda nb, ms: f"{nb / ms / 1e6 / PEAK_GBS * 100:5.1f}"
            for n in (16384, 16384 + 64, 16384 + 128, 16384 + 512, 16384 + 1024, 16384 - 64, 12288, 8192 + 64, 8192):
                pool = torch.empty(2 * n * n, device=dev)
                src = wl.fill_uniform(pool[:n * n], 1002).view(n, n)
                dst = pool[n * n:].view(n, n)
                sink = torch.empty(8 * cus * 4, device=dev)
                nb = n * n * 4
                reads = [pct(nb, _time(lambda: wl.probe_pattern("tile_read", src, None, sink, int(cus * wg)), args.steps, settle_ms=10.0)) for wg in (1, 1.5, 2)]
                writes = [pct(nb, _time(lambda: wl.probe_pattern("tile_write", None, None, dst, int(cus * wg)), args.steps, settle_ms=10.0)) for wg in (0.5, 1, 1.5)]
                kernel = pct(2 * nb, _time(lambda: wl.strided_transpose(src, dst, 0), args.steps, settle_ms=20.0))
                if not torch.equal(dst, src.t()):
                    sys.exit(f"transposition of {n} x {n} is wrong")
                print(f"n = {n:5d} (row pitch {4 * n} B): tile reads alone {' / '.join(reads)} % at (1, 1.5, 2) workgroups per CU; tile writes alone "
                      f"{' / '.join(writes)} % at (0.5, 1, 1.5); cudadma_strided_transpose variant 0 {kernel} %", flush=True)
                del pool, src, dst
        elif name == "channel_hash":
            # reads the half of a 1 GiB buffer whose 256-byte granules have even parity under one, two or three address bits:
            # a parity that picks half of the memory channels halves the rate
            import itertools
            buf = wl.fill_uniform(torch.empty(1 << 28, device=dev), 9)
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            groups = int(cus * 1.5)
            sink = torch.empty(groups * 4, device=dev)
            bits = range(22)                                    # granule-index bits 0..21 = address bits 8..29
            def rate(mask):
                # the better of two measurements: one launch in a few thousand is held up by something else on the machine
                ms = min(_time(lambda: wl.probe_pattern("masked_read", buf, None, sink, groups, n_records=mask), 5, warmup=2, settle_ms=0.0)
                         for _ in range(2))
                return (1 << 29) / ms / 1e6
            for _ in range(20):
                rate(1 << 21)
            print("# GB/s of the half of 1 GiB chosen by the parity of the address bits named")
            for b in bits:
                print(f"bit {b + 8:2d}: {rate(1 << b):6.0f}", flush=True)
            found = []
            for k in (2, 3):
                for combo in itertools.combinations(bits, k):
                    mask = sum(1 << b for b in combo)
                    found.append((rate(mask), combo))
            found.sort()
            print("# the 24 slowest of the 1771 pairs and triples, and the median")
            for r, combo in found[:24]:
                print(f"bits {' ^ '.join(str(b + 8) for b in combo):14s}: {r:6.0f}", flush=True)
            print(f"median: {found[len(found) // 2][0]:6.0f}")
            del buf
        elif name == "settle":
            # what the first launches after an idle phase cost, and whether the shader clock has anything to do with it: after a
            # second without GPU work, launches of one kernel back to back, each between two events, a clock probe after each
            import time
            n = 16384
            pool = torch.empty(2 * n * n, device=dev)
            src = wl.fill_uniform(pool[:n * n], 1002).view(n, n)
            dst = pool[n * n:].view(n, n)
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            kernels = (("transposition (variant 0)", lambda: wl.strided_transpose(src, dst, 0), 2 * n * n * 4),
                       ("copy_nontemporal yardstick, 4 workgroups per CU", lambda: wl.probe_memory("copy_nontemporal", src.view(-1), dst.view(-1), cus * 4), 2 * n * n * 4),
                       ("read_nontemporal yardstick, 1.5 workgroups per CU", lambda: wl.probe_memory("read_nontemporal", src.view(-1), None, int(cus * 1.5)), n * n * 4))
            launches = 80
            for label, fn, nbytes in kernels:
                ticks = torch.zeros((launches, 2), dtype=torch.int64, device=dev)
                events = [torch.cuda.Event(enable_timing=True) for _ in range(launches + 1)]
                torch.cuda.synchronize()
                time.sleep(1.0)
                events[0].record()
                for i in range(launches):
                    fn()
                    events[i + 1].record()
                    wl.probe_clock(ticks[i], 2048)          # a few microseconds
                torch.cuda.synchronize()
                t = ticks.cpu()
                print(f"# {label}: launch, ms since the first launch, ms of the launch (incl. the clock probe behind it), % of 8 TB/s, shader clock in MHz")
                at = 0.0
                for i in range(launches):
                    ms = events[i].elapsed_time(events[i + 1])
                    mhz = 100.0 * t[i, 0].item() / max(1, t[i, 1].item())
                    if i < 12 or i % 4 == 0:
                        print(f"{i:3d}  {at:8.3f}  {ms:.4f}  {nbytes / ms / 1e6 / PEAK_GBS * 100:5.1f}  {mhz:7.0f}", flush=True)
                    at += ms
            del pool
        elif name == "queue_depth":
            if args.config not in QUEUE_CONFIGS:
                sys.exit("--config must be one of: " + ", ".join(QUEUE_CONFIGS))
            what, shape = QUEUE_CONFIGS[args.config]
            m = (1 << 30) // 4
            pool = torch.empty(2 * m, device=dev)              # destination exactly 1 GiB behind the source
            src, dst = wl.fill_uniform(pool[:m], 1002), pool[m:]
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            if what == "transpose":
                wl.set_tuning("transpose_split", shape["transpose_split"])
                wl.set_tuning("transpose_workgroups", cus * shape["transpose_workgroups"])
                fn = lambda: wl.strided_transpose(src.view(16384, 16384), dst.view(16384, 16384), wl.TRANSPOSE_SPLIT_VARIANT)
                nbytes = 2 * m * 4
            elif what == "pattern":
                mode, piece, wg, grouped = shape
                wl.set_tuning("probe_piece_bytes", piece)
                wl.set_tuning("probe_xcd_group", grouped)
                if mode == "scatter":
                    recs = 4 << 20
                    records = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, device=dev), 1006)
                    perm = wl.fill_permutation(torch.empty(recs, dtype=torch.int32, device=dev), 1006)
                    table = torch.empty(recs * wl.REC_FLOATS, device=dev)
                    fn = lambda: wl.probe_pattern("scatter", records, perm, table, int(cus * wg))
                    nbytes = recs * 260
                elif mode.startswith("gather"):
                    del pool
                    size = mode.rsplit("_", 1)[-1]                      # records in the table: _small = 4 Mi, _<k>Mi, else 32 Mi
                    recs = (4 << 20) if size == "small" else (int(size[:-2]) << 20) if size.endswith("Mi") else (32 << 20)
                    n_idx = 32 << 20
                    pool = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, device=dev), 1003)
                    idx = wl.fill_indices(torch.empty(n_idx, dtype=torch.int32, device=dev), recs, 1003)
                    out = torch.empty(n_idx // wl.RECS_PER_TILE * wl.REC_FLOATS, device=dev)
                    if mode.startswith("gather_dma"):
                        fn = lambda: wl.gather_rowsum(pool, idx, out, 0)
                    else:
                        fn = lambda: wl.probe_pattern("gather_xor", pool, idx, out, int(cus * wg))
                    nbytes = n_idx * 132 + out.numel() * 4
                elif mode == "tile_read":
                    sink = torch.empty(8 * cus * 4, device=dev)
                    fn = lambda: wl.probe_pattern("tile_read", src.view(16384, 16384), None, sink, int(cus * wg))
                    nbytes = m * 4
                else:
                    fn = lambda: wl.probe_pattern(mode, None, None, dst.view(16384, 16384), int(cus * wg))
                    nbytes = m * 4
            elif what == "perf_sequential":
                groups, elmt = 2 * cus, 16 * 1024
                lq = wl.LOAD_CACHE_STREAMING if shape == "LOAD_CACHE_STREAMING" else wl.LOAD_CACHE_ALL
                fn = lambda: wl.perf_sequential(src, elmt, 4, wl.BUFFERING_MANUAL, (m * 4) // (groups * elmt), groups, None, lq, wl.STORE_LDS)
                nbytes = m * 4
            else:
                s_, d_ = (None if what.startswith("write") else src), (None if what.startswith("read") else dst)
                fn = lambda: wl.probe_memory(what, s_, d_, int(cus * shape))
                nbytes = (m * 4 if s_ is not None else 0) + (m * 4 if d_ is not None else 0)
            ms = _time(fn, args.steps, warmup=2, settle_ms=0.0)
            print(f"queue_depth {args.config:22s} {ms:8.4f} ms  {nbytes / ms / 1e6:7.0f} GB/s  {100 * nbytes / ms / 1e6 / PEAK_GBS:5.1f}%", flush=True)
            wl.set_tuning("transpose_split", 0)
            wl.set_tuning("transpose_workgroups", 0)
            wl.set_tuning("probe_piece_bytes", 0)
            wl.set_tuning("probe_xcd_group", 0)
            del pool
        elif name == "two_streams":
            # a read-only and a write-only kernel, 1 GiB each, side by side on two streams: do two kernels that each issue one
            # kind of request pass the copy, whose every wavefront issues both?
            m = (1 << 30) // 4
            pool = torch.empty(2 * m, device=dev)
            src, dst = wl.fill_uniform(pool[:m], 1002), pool[m:]
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()

            def pair(read_wg, write_wg, reps):
                torch.cuda.synchronize()
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                s1.wait_event(a)
                s2.wait_event(a)
                for _ in range(reps):
                    with torch.cuda.stream(s1):
                        wl.probe_memory("read_nontemporal", src, None, int(cus * read_wg))
                    with torch.cuda.stream(s2):
                        wl.probe_memory("write", None, dst, int(cus * write_wg))
                e1, e2 = torch.cuda.Event(), torch.cuda.Event()
                e1.record(s1)
                e2.record(s2)
                torch.cuda.current_stream().wait_event(e1)
                torch.cuda.current_stream().wait_event(e2)
                b.record()
                torch.cuda.synchronize()
                return a.elapsed_time(b) / reps

            pair(1.5, 0.5, 40)
            ms = _time(lambda: wl.probe_memory("copy_nontemporal", src, dst, 4 * cus), args.steps)
            print(f"two_streams  one copy kernel, 4 wg/cu                        {ms:8.4f} ms  {100 * 2 * m * 4 / ms / 1e6 / PEAK_GBS:5.1f}%")
            for read_wg in (0.5, 0.75, 1, 1.5, 2):
                for write_wg in (0.25, 0.5, 1, 2):
                    ms = pair(read_wg, write_wg, args.steps)
                    print(f"two_streams  read {read_wg:4} wg/cu beside write {write_wg:4} wg/cu, per pair  {ms:8.4f} ms  "
                          f"{100 * 2 * m * 4 / ms / 1e6 / PEAK_GBS:5.1f}%", flush=True)
            del pool
        elif name == "scatter":
            recs = 4 << 20
            records = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, device=dev), 1006)
            perm = wl.fill_permutation(torch.empty(recs, dtype=torch.int32, device=dev), 1006)
            table = torch.empty(recs * wl.REC_FLOATS, device=dev)
            for v in wl.variants(wl.SCATTER):
                print(f"# scatter variant {v}: {wl.variant_name(wl.SCATTER, v)}")
                for wg in wgs:
                    wl.set_workgroups_per_cu(wg)
                    _row(name, v, wg, _time(lambda: wl.scatter_copy(records, perm, table, v), args.steps), recs * 260)
        elif name == "halo":
            g = 512
            gi = wl.fill_uniform(torch.empty((g + 8) ** 3, device=dev), 1004).view(g + 8, g + 8, g + 8)
            go = torch.empty(g, g, g, device=dev)
            for v in wl.variants(wl.HALO):
                print(f"# halo variant {v}: {wl.variant_name(wl.HALO, v)}")
                for zc in (0, 128, 256, 512):
                    wl.set_tuning("stencil_zchunk", zc)
                    ms = _time(lambda: wl.halo_stencil(gi, go, v), args.steps)
                    gbs = 2 * g ** 3 * 4 / ms / 1e6
                    print(f"{name:10s} variant {v}  zchunk {zc:3d}  {ms:9.4f} ms  {gbs:8.0f} GB/s  {100 * gbs / PEAK_GBS:5.1f}%",
                          flush=True)
            wl.set_tuning("stencil_zchunk", 0)
        elif name == "gemm":
            # every variant at 4096^3 and 8192^3, torch.matmul (hipBLASLt) on the same tensors beside them
            for n in (4096, 8192):
                a = torch.randn(n, n, device=dev).to(torch.bfloat16)
                b = torch.randn(n, n, device=dev).to(torch.bfloat16)
                c = torch.empty(n, n, device=dev)
                for v in wl.variants(wl.GEMM)[1:]:
                    ms = _time(lambda: wl.gemm_bf16(a, b, c, v), args.steps, settle_ms=10.0)
                    print(f"gemm {n}^3  variant {v}  {ms:9.4f} ms  {2.0 * n ** 3 / ms / 1e9:8.1f} TFLOP/s", flush=True)
                ms = _time(lambda: torch.matmul(a, b), args.steps, settle_ms=10.0)
                print(f"gemm {n}^3  torch.matmul  {ms:9.4f} ms  {2.0 * n ** 3 / ms / 1e9:8.1f} TFLOP/s", flush=True)
                del a, b, c
        elif name == "perf_sequential":
            # src/perf/sequential/param_sweep.py:27-58: element size x DMA wavefronts x workgroups per CU x
            # buffering; a launch reads 1 GiB whatever the point (loop count follows from that).  On top of the
            # reference's space: the cache qualifier of the loads and how the bytes reach LDS.
            src = wl.fill_uniform(torch.empty(1 << 28, device=dev), 1001)
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            quals = (("LOAD_CACHE_ALL, STORE_WRITE_BACK (the reference's defaults)", wl.LOAD_CACHE_ALL, wl.STORE_WRITE_BACK),
                     ("LOAD_CACHE_STREAMING, STORE_LDS", wl.LOAD_CACHE_STREAMING, wl.STORE_LDS),
                     ("LOAD_CACHE_ALL, STORE_LDS_DIRECT", wl.LOAD_CACHE_ALL, wl.STORE_LDS_DIRECT),
                     ("LOAD_CACHE_STREAMING, STORE_LDS_DIRECT", wl.LOAD_CACHE_STREAMING, wl.STORE_LDS_DIRECT))
            for label, lq, sq in quals:
                print(f"# {label}: read bandwidth into LDS, GB/s (1 GiB per launch); columns: buffering none / single / double / manual")
                for elmt in (32, 128, 512, 2048, 4096, 8192, 16384):
                    for waves in (1, 2, 4):
                        for wg in wgs if wgs != [0] else [4]:
                            wg = wg or 4
                            groups = cus * wg
                            loops = max(1, (1 << 30) // (groups * elmt))
                            cells = []
                            for b in range(4):
                                run = lambda: wl.perf_sequential(src, elmt, waves, b, loops, groups, None, lq, sq)
                                nbytes = run()
                                ms = _time(run, args.steps, settle_ms=5.0)
                                cells.append(f"{nbytes / ms / 1e6:7.0f}")
                            print(f"elmt {elmt:6d} B  dma waves {waves}  wg/cu {wg:2d}  loops {loops:6d}  " + " ".join(cells), flush=True)
        elif name == "saxpy":
            # bytes as the reference's driver counts them: x read, y read, y written (saxpy_cudaDMA.cu:192)
            n = 1 << 28
            x = wl.fill_uniform(torch.empty(n, device=dev), 11)
            y = wl.fill_uniform(torch.empty(n, device=dev), 12)
            for v in range(ex.num_variants(ex.SAXPY)):
                print(f"# saxpy variant {v}: {ex.variant_name(ex.SAXPY, v)}")
                for wg in wgs:
                    wl.set_workgroups_per_cu(wg)
                    _row(name, v, wg, _time(lambda: ex.saxpy(1e-3, x, y, v), args.steps), 3 * n * 4)
        elif name == "sgemv":
            n = m = 16384
            a = wl.fill_uniform(torch.empty(m * n, device=dev), 21).view(m, n)
            x = wl.fill_uniform(torch.empty(m, device=dev), 22)
            y = torch.empty(n, device=dev)
            for v in range(ex.num_variants(ex.SGEMV)):
                print(f"# sgemv variant {v}: {ex.variant_name(ex.SGEMV, v)}")
                _row(name, v, 0, _time(lambda: ex.sgemv(1.0, a, x, y, variant=v), args.steps), (m * n + m + n) * 4)
        elif name == "stencil2d":
            # the reference's directed size (params_directed.h): 960 x 160 x 200 float2, tiles of 32 x 4;
            # bytes as its driver counts them: tile plus halo read, tile written (cudaDMA_stencil2D.cu:225-232)
            dimx, dimy, dimz, r = 960, 160, 200, ex.STENCIL2D_RADIUS
            shape = (dimz + 2 * r, dimy + 2 * r, dimx + 2 * r, 2)
            src = wl.fill_uniform(torch.empty(shape, device=dev).view(-1), 31).view(shape)
            dst = torch.zeros(shape, device=dev)
            tiles = (dimx // 32) * (dimy // 4)
            issued = tiles * dimz * ((4 + 2 * r) * (32 + 2 * r) + 4 * 32) * 8
            for v in range(ex.num_variants(ex.STENCIL2D)):
                print(f"# stencil2d variant {v}: {ex.variant_name(ex.STENCIL2D, v)}")
                _row(name, v, 0, _time(lambda: ex.stencil2d(src, dst, v), args.steps), issued)
        else:
            sys.exit(f"unknown workload {name}")
    wl.set_workgroups_per_cu(0)


if __name__ == "__main__":
    main()
