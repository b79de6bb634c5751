"""Turns rocprofv3 output of bench.py into profiles/counters.json (what bench.py reads its counter-derived
fields from) and a table for the text summaries under profiles/.

Expected layout, one directory per pattern of bench.py (`--only <pattern>`), one sub-directory per collection:

    <root>/<pattern>/trace/   rocprofv3 --kernel-trace --stats --output-format csv -d <root>/<pattern>/trace -o b -- python3 bench.py --only <pattern> --steps 20 --no-cpu-baseline > <root>/<pattern>/trace.json
    <root>/<pattern>/fetch/   rocprofv3 --pmc FETCH_SIZE --output-format csv -d ... -o b -- python3 bench.py --only <pattern>,plain_copy --steps 3 --warmup 1 --no-cpu-baseline
    <root>/<pattern>/write/   rocprofv3 --pmc WRITE_SIZE ...                                   (same command)
    <root>/<pattern>/lds/     rocprofv3 --pmc SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE ...       (optional)
    <root>/<pattern>/mfma/    rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CU_CYCLES ...   (optional, the GEMM)

FETCH_SIZE and WRITE_SIZE (KiB per dispatch) are scaled by what the same counters read, in the same run, for
the library's plain copy of 1 GiB (`plain_copy_kernel`: 1 048 576 KiB read and as many written).

    python -m cudadma_amd.profile_summary <root> > table.md      # writes profiles/counters.json

Two further tables, printed only:

    python -m cudadma_amd.profile_summary --series <dir>     every dispatch of a rocprofv3 --kernel-trace run in order of
                                                             start: start time, duration, gap to the one before, kernel
    python -m cudadma_amd.profile_summary --queue <root>     counters of launch shapes that differ in the work in flight:
        <root>/<config>/plain.txt   output of  python3 -m cudadma_amd.sweep queue_depth --config <config>   (no profiler)
        <root>/<config>/p<i>/       rocprofv3 --pmc <at most 4 TCC_, 4 TCP_, 2 TA_, 2 GRBM_, 8 SQ_ counters> --output-format csv
                                    -d <root>/<config>/p<i> -o q -- python3 -m cudadma_amd.sweep queue_depth --config <config> --steps 3
"""
import csv
import glob
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
COPY_KERNEL = "plain_copy_kernel"
COPY_KIB = 1048576.0          # the calibration copy moves 1 GiB each way


def _rows(directory, suffix):
    files = glob.glob(os.path.join(directory, "**", f"*{suffix}"), recursive=True)
    for path in files:
        with open(path, newline="") as f:
            yield from csv.DictReader(f)


def _matches(kernel_name, wanted):
    # rocprofv3 prints "void (anonymous namespace)::name<args>(params)"; compare without the namespace and the parameters
    flat = kernel_name.replace("(anonymous namespace)::", "")
    return wanted.replace("(anonymous namespace)::", "") in flat


def durations_us(directory, kernel, last=20):
    """Average, min, max duration (us) over the last `last` dispatches of `kernel`, and the dispatch count."""
    d = [(int(r["Start_Timestamp"]), (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
         for r in _rows(directory, "_kernel_trace.csv") if _matches(r["Kernel_Name"], kernel)]
    if not d:
        return None
    d.sort()
    tail = [x[1] for x in d[-last:]]
    return {"dispatches": len(d), "avg_us": sum(tail) / len(tail), "min_us": min(tail), "max_us": max(tail)}


def stats_row(directory, kernel):
    """rocprofv3's own --stats line for `kernel`: calls and average duration over every dispatch of the run."""
    for r in _rows(directory, "_kernel_stats.csv"):
        if _matches(r["Name"], kernel):
            return {"stats_calls": int(r["Calls"]), "stats_avg_us": round(float(r["AverageNs"]) / 1e3, 2)}
    return {}


def counter_means(directory, kernel):
    """Mean value per dispatch of every counter collected for `kernel`."""
    acc = {}
    for r in _rows(directory, "_counter_collection.csv"):
        if _matches(r["Kernel_Name"], kernel):
            acc.setdefault(r["Counter_Name"], []).append(float(r["Counter_Value"]))
    return {k: sum(v) / len(v) for k, v in acc.items()}


def summarise(root):
    import bench
    out = {"patterns": {}, "calibration": {}}
    try:
        out["collected_at_commit"] = subprocess.check_output(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], text=True).strip()
    except (OSError, subprocess.CalledProcessError):
        out["collected_at_commit"] = None
    for name in sorted(os.listdir(root)):
        pdir = os.path.join(root, name)
        kernel = bench.PATTERN_KERNELS.get(name)
        if not os.path.isdir(pdir) or kernel is None:
            continue
        row = {"kernel": kernel}
        algorithmic = None
        tj = os.path.join(pdir, "trace.json")
        if os.path.exists(tj):
            try:
                line = [l for l in open(tj) if l.startswith("{")][-1]
                res = json.loads(line)
                src = res.get("patterns", {}).get(name) or {}
                if name.startswith("gemm"):
                    g = res.get("gemm", {})
                    src = g if name == "gemm" else g.get("warp_specialised", {})
                    row["flop"] = src.get("flop")
                    row["hip_event_ms"] = src.get("ms")
                else:
                    algorithmic = src.get("algorithmic_bytes")
                    row["algorithmic_bytes"] = algorithmic
                    row["hip_event_ms"] = src.get("ms")
            except (IndexError, ValueError):
                pass
        t = durations_us(os.path.join(pdir, "trace"), kernel) if os.path.isdir(os.path.join(pdir, "trace")) else None
        if t:
            row.update({k: round(v, 2) if isinstance(v, float) else v for k, v in t.items()})
            row.update(stats_row(os.path.join(pdir, "trace"), kernel))
            if algorithmic:
                row["GB/s_at_avg"] = round(algorithmic / t["avg_us"] / 1e3, 1)
            if row.get("flop"):
                row["TFLOP/s_at_avg"] = round(row["flop"] / t["avg_us"] / 1e6, 1)
        scaled = {}
        for kind, counter in (("fetch", "FETCH_SIZE"), ("write", "WRITE_SIZE")):
            cdir = os.path.join(pdir, kind)
            if not os.path.isdir(cdir):
                continue
            mine, copy = counter_means(cdir, kernel).get(counter), counter_means(cdir, COPY_KERNEL).get(counter)
            if mine is None or not copy:
                continue
            factor = COPY_KIB / copy
            row[f"{counter}_KiB"] = round(mine, 1)
            row[f"{counter}_KiB_plain_copy"] = round(copy, 1)
            row[f"{counter}_scale"] = round(factor, 5)
            scaled[kind] = mine * factor * 1024.0
            out["calibration"].setdefault(counter, []).append(round(copy, 1))
        if len(scaled) == 2:
            row["read_bytes"] = int(round(scaled["fetch"]))
            row["written_bytes"] = int(round(scaled["write"]))
            row["traffic_bytes"] = row["read_bytes"] + row["written_bytes"]
            if algorithmic:
                row["traffic_over_algorithmic"] = round(row["traffic_bytes"] / algorithmic, 4)
        ldir = os.path.join(pdir, "lds")
        if os.path.isdir(ldir):
            c = counter_means(ldir, kernel)
            if c.get("SQ_LDS_IDX_ACTIVE"):
                row["SQ_LDS_BANK_CONFLICT"] = round(c.get("SQ_LDS_BANK_CONFLICT", 0.0), 1)
                row["SQ_LDS_IDX_ACTIVE"] = round(c["SQ_LDS_IDX_ACTIVE"], 1)
                row["lds_bank_conflict_ratio"] = round(c.get("SQ_LDS_BANK_CONFLICT", 0.0) / c["SQ_LDS_IDX_ACTIVE"], 4)
        mdir = os.path.join(pdir, "mfma")
        if os.path.isdir(mdir):
            c = counter_means(mdir, kernel)
            if c.get("SQ_BUSY_CU_CYCLES"):
                # matrix-core busy cycles are summed over the four SIMDs of a compute unit
                row["SQ_VALU_MFMA_BUSY_CYCLES"] = round(c.get("SQ_VALU_MFMA_BUSY_CYCLES", 0.0), 1)
                row["SQ_BUSY_CU_CYCLES"] = round(c["SQ_BUSY_CU_CYCLES"], 1)
                row["mfma_busy"] = round(c.get("SQ_VALU_MFMA_BUSY_CYCLES", 0.0) / 4.0 / c["SQ_BUSY_CU_CYCLES"], 4)
                for extra in ("SQ_WAIT_INST_ANY", "SQ_LDS_IDX_ACTIVE", "SQ_LDS_BANK_CONFLICT", "SQ_WAVE_CYCLES"):
                    if extra in c:
                        row[extra] = round(c[extra], 1)
        out["patterns"][name] = row
    return out


def markdown(summary):
    cols = ["kernel", "dispatches", "avg_us", "min_us", "max_us", "stats_avg_us", "hip_event_ms", "GB/s_at_avg", "TFLOP/s_at_avg", "FETCH_SIZE_KiB", "WRITE_SIZE_KiB",
            "traffic_bytes", "traffic_over_algorithmic", "lds_bank_conflict_ratio", "mfma_busy"]
    lines = ["| pattern | " + " | ".join(cols) + " |", "|---|" + "---|" * len(cols)]
    for name, row in summary["patterns"].items():
        lines.append(f"| {name} | " + " | ".join(str(row.get(c, "")) for c in cols) + " |")
    return "\n".join(lines)


def dispatch_series(directory):
    """Markdown table of every dispatch of a kernel-trace run, in order of start."""
    rows = sorted(_rows(directory, "_kernel_trace.csv"), key=lambda r: int(r["Start_Timestamp"]))
    if not rows:
        sys.exit(f"no *_kernel_trace.csv under {directory}")
    t0, prev_end = int(rows[0]["Start_Timestamp"]), None
    lines = ["| # | start, ms | duration, us | idle before, us | kernel |", "|---|---|---|---|---|"]
    for i, r in enumerate(rows):
        s_, e_ = int(r["Start_Timestamp"]), int(r["End_Timestamp"])
        name = r["Kernel_Name"].replace("(anonymous namespace)::", "").replace("void ", "").split("(")[0]
        gap = (s_ - prev_end) / 1e3 if prev_end is not None else 0.0
        lines.append(f"| {i} | {(s_ - t0) / 1e6:.3f} | {(e_ - s_) / 1e3:.1f} | {gap:.1f} | `{name}` |")
        prev_end = e_
    return "\n".join(lines)


# derived rows of the queue table: (label, function of the per-dispatch counter means)
def _ratio(a, b):
    return lambda c: c[a] / c[b] if c.get(b) else None


_QUEUE_DERIVED = (
    ("ms per launch (no profiler)", lambda c: c.get("ms")),
    ("% of 8 TB/s (no profiler)", lambda c: c.get("pct")),
    ("read requests L2 -> fabric (128 B each), millions", lambda c: c["TCC_EA0_RDREQ_sum"] / 1e6 if "TCC_EA0_RDREQ_sum" in c else None),
    ("write requests L2 -> fabric (64 B each), millions", lambda c: c["TCC_EA0_WRREQ_sum"] / 1e6 if "TCC_EA0_WRREQ_sum" in c else None),
    ("read latency L2 -> fabric -> L2, L2 cycles (RDREQ_LEVEL / RDREQ)", _ratio("TCC_EA0_RDREQ_LEVEL_sum", "TCC_EA0_RDREQ_sum")),
    ("write latency L2 -> fabric, L2 cycles (WRREQ_LEVEL / WRREQ)", _ratio("TCC_EA0_WRREQ_LEVEL_sum", "TCC_EA0_WRREQ_sum")),
    ("reads outstanding per L2 channel (RDREQ_LEVEL / TCC_CYCLE)", _ratio("TCC_EA0_RDREQ_LEVEL_sum", "TCC_CYCLE_sum")),
    ("writes outstanding per L2 channel (WRREQ_LEVEL / TCC_CYCLE)", _ratio("TCC_EA0_WRREQ_LEVEL_sum", "TCC_CYCLE_sum")),
    ("cycles a read waited for a DRAM credit, per read (RDREQ_DRAM_CREDIT_STALL / RDREQ)", _ratio("TCC_EA0_RDREQ_DRAM_CREDIT_STALL_sum", "TCC_EA0_RDREQ_sum")),
    ("cycles a write waited for a DRAM credit, per write (WRREQ_DRAM_CREDIT_STALL / WRREQ)", _ratio("TCC_EA0_WRREQ_DRAM_CREDIT_STALL_sum", "TCC_EA0_WRREQ_sum")),
    ("L2 tag stall cycles per L2 request (TAG_STALL / REQ)", _ratio("TCC_TAG_STALL_sum", "TCC_REQ_sum")),
    ("L1 read latency seen by the L1, cycles (TCP_TCC_READ_REQ_LATENCY / READ_REQ)", _ratio("TCP_TCC_READ_REQ_LATENCY_sum", "TCP_TCC_READ_REQ_sum")),
    ("L1 write latency, cycles (TCP_TCC_WRITE_REQ_LATENCY / WRITE_REQ)", _ratio("TCP_TCC_WRITE_REQ_LATENCY_sum", "TCP_TCC_WRITE_REQ_sum")),
    ("address unit stalled by the L1, share of its busy time (TA_ADDR_STALLED_BY_TC / (256 x GRBM_TA_BUSY / 8))",
     lambda c: c["TA_ADDR_STALLED_BY_TC_CYCLES_sum"] / (32.0 * c["GRBM_TA_BUSY"]) if c.get("GRBM_TA_BUSY") and "TA_ADDR_STALLED_BY_TC_CYCLES_sum" in c else None),
    ("L1 stalled by the router between it and the L2, million cycles (TCP_TCR_TCP_STALL)", lambda c: c["TCP_TCR_TCP_STALL_CYCLES_sum"] / 1e6 if "TCP_TCR_TCP_STALL_CYCLES_sum" in c else None),
    ("translation misses in the L1 TLB (UTCL1_TRANSLATION_MISS)", lambda c: c.get("TCP_UTCL1_TRANSLATION_MISS_sum")),
    ("translation requests per memory instruction (UTCL1_REQUEST / (VMEM_RD + VMEM_WR))",
     lambda c: c["TCP_UTCL1_REQUEST_sum"] / (c.get("SQ_INSTS_VMEM_RD", 0) + c.get("SQ_INSTS_VMEM_WR", 0)) if c.get("TCP_UTCL1_REQUEST_sum") and (c.get("SQ_INSTS_VMEM_RD", 0) + c.get("SQ_INSTS_VMEM_WR", 0)) else None),
    ("L1 TLB: cycles stalled at its limit of requests in flight, millions (UTCL1_STALL_INFLIGHT_MAX)",
     lambda c: c["TCP_UTCL1_STALL_INFLIGHT_MAX_sum"] / 1e6 if "TCP_UTCL1_STALL_INFLIGHT_MAX_sum" in c else None),
    ("L2 TLB busy, thousand cycles (GRBM_UTCL2_BUSY)", lambda c: c["GRBM_UTCL2_BUSY"] / 1e3 if "GRBM_UTCL2_BUSY" in c else None),
    ("vector memory instructions in flight, relative figure (SQ_INST_LEVEL_VMEM / SQ_BUSY_CYCLES)",
     _ratio("SQ_INST_LEVEL_VMEM", "SQ_BUSY_CYCLES")),
    ("wavefront cycles waiting for anything, share (SQ_WAIT_ANY / SQ_WAVE_CYCLES)", _ratio("SQ_WAIT_ANY", "SQ_WAVE_CYCLES")),
    ("wavefront cycles waiting to issue, share (SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES)", _ratio("SQ_WAIT_INST_ANY", "SQ_WAVE_CYCLES")),
)


def queue_table(root, configs=None):
    """Markdown table: one column per launch shape under <root>, one row per derived figure."""
    import collections
    configs = configs or sorted(d for d in os.listdir(root) if os.path.isdir(os.path.join(root, d)))
    table = collections.OrderedDict()
    for cfg in configs:
        vals = {}
        for path in glob.glob(os.path.join(root, cfg, "p*", "**", "*counter_collection.csv"), recursive=True):
            with open(path, newline="") as f:
                rows = list(csv.DictReader(f))
            # the kernel under test: the most frequent one that is not an input generator
            names = collections.Counter(r["Kernel_Name"] for r in rows if "fill_" not in r["Kernel_Name"])
            if not names:
                continue
            kernel = names.most_common(1)[0][0]
            per = collections.defaultdict(list)
            for r in rows:
                if r["Kernel_Name"] == kernel:
                    per[r["Counter_Name"]].append(float(r["Counter_Value"]))
            for c, v in per.items():
                vals[c] = sum(v[-3:]) / len(v[-3:])          # the timed launches are the last three
        try:
            with open(os.path.join(root, cfg, "plain.txt")) as f:
                words = [l for l in f if l.startswith("queue_depth")][-1].split()
            vals["ms"], vals["pct"] = float(words[2]), float(words[6].rstrip("%"))
        except (OSError, IndexError, ValueError):
            pass
        table[cfg] = vals
    lines = ["| | " + " | ".join(table) + " |", "|---|" + "---|" * len(table)]
    for label, fn in _QUEUE_DERIVED:
        cells = []
        for cfg, vals in table.items():
            try:
                v = fn(vals)
            except KeyError:
                v = None
            cells.append("" if v is None else (f"{v:.4g}" if abs(v) < 1e5 else f"{v:.0f}"))
        if any(cells):
            lines.append(f"| {label} | " + " | ".join(cells) + " |")
    return "\n".join(lines)


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    if len(argv) >= 2 and argv[0] == "--series":
        print(dispatch_series(argv[1]))
        return
    if len(argv) >= 2 and argv[0] == "--queue":
        print(queue_table(argv[1], argv[2:] or None))
        return
    if len(argv) != 1:
        sys.exit(__doc__)
    summary = summarise(argv[0])
    with open(os.path.join(ROOT, "profiles", "counters.json"), "w") as f:
        json.dump(summary, f, indent=1, sort_keys=True)
        f.write("\n")
    print(markdown(summary))


if __name__ == "__main__":
    main()
