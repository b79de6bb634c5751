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


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    if len(argv) != 1:
        sys.exit(__doc__)
    summary = summarise(argv[0])
    with open(os.path.join(ROOT, "profiles", "counters.json"), "w") as f:
        json.dump(summary, f, indent=1, sort_keys=True)
        f.write("\n")
    print(markdown(summary))


if __name__ == "__main__":
    main()
