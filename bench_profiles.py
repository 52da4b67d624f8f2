#!/usr/bin/env python3
"""Turns rocprofv3 output of `bench.py` runs into the summaries under profiles/.

bench.py cannot read hardware counters from inside its own process, so the per-kernel HBM traffic
and the instruction counters come from separate rocprofv3 runs of the same script; this tool
reads their CSV files and writes a short markdown table and, for the traffic, a JSON record that
bench.py quotes as `roofline.traffic` (with the commit the counters were taken at).

    # on the MI355X box, repository root (each counter set in a run of its own; W = cfg1 .. cfg4, dense):
    export TMPDIR=/tmp
    rocprofv3 --kernel-trace --stats --output-format csv -d out/W/prof -o bench -- \\
        python3 bench.py --workload W --steps 20 --warmup 5 --no-cpu-baseline
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d out/W/pmc_fetch -o f -- \\
        python3 bench.py --workload W --steps 2 --warmup 1 --no-cpu-baseline --copy-probe > out/W/pmc_fetch.json
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d out/W/pmc_write -o w -- \\
        python3 bench.py --workload W --steps 2 --warmup 1 --no-cpu-baseline --copy-probe
    rocprofv3 --pmc SQ_WAVES SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_INSTS_VALU SQ_ACTIVE_INST_VALU SQ_INSTS_SALU \\
        SQ_INSTS_LDS SQ_LDS_BANK_CONFLICT --output-format csv -d out/W/pmc_sq -o s -- \\
        python3 bench.py --workload W --steps 2 --warmup 1 --no-cpu-baseline

    # anywhere the CSV files are (the commit is read from git when --commit is not given):
    python3 bench_profiles.py stats   out/W/prof --workload W --name W_kernel_stats
    python3 bench_profiles.py traffic out/W/pmc_fetch out/W/pmc_write --bench-json out/W/pmc_fetch.json \\
        --workload W --name W_hbm_traffic_per_kernel
    python3 bench_profiles.py sq      out/W/pmc_sq out/W/prof --workload W --name W_sq_counters_per_kernel
    # (optional, `mem`: vector-memory instructions and L2 atomics per kernel; its command is in the summary it writes)
"""
import argparse
import collections
import csv
import glob
import json
import os
import re
import statistics
import subprocess
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
PROFILES = os.path.join(ROOT, "profiles")

# the commands whose output this tool reads; {dir} is the directory that the tool was given
STATS_CMD = ("rocprofv3 --kernel-trace --stats --output-format csv -d {dir} -o bench -- "
             "python3 bench.py --workload {workload} --steps 20 --warmup 5 --no-cpu-baseline")
FETCH_CMD = ("rocprofv3 --pmc FETCH_SIZE --output-format csv -d {dir} -o f -- "
             "python3 bench.py --workload {workload} --steps 2 --warmup 1 --no-cpu-baseline --copy-probe")
WRITE_CMD = ("rocprofv3 --pmc WRITE_SIZE --output-format csv -d {dir} -o w -- "
             "python3 bench.py --workload {workload} --steps 2 --warmup 1 --no-cpu-baseline --copy-probe")
SQ_CMD = ("rocprofv3 --pmc SQ_WAVES SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_INSTS_VALU SQ_ACTIVE_INST_VALU SQ_INSTS_SALU "
          "SQ_INSTS_LDS SQ_LDS_BANK_CONFLICT --output-format csv -d {dir} -o s -- "
          "python3 bench.py --workload {workload} --steps 2 --warmup 1 --no-cpu-baseline")


MEM_CMD = ("rocprofv3 --pmc SQ_WAVES SQ_INSTS_VMEM_WR SQ_INSTS_VMEM_RD SQ_INSTS_BRANCH TCC_ATOMIC_sum "
           "TCP_TCC_ATOMIC_WITHOUT_RET_REQ_sum --output-format csv -d {dir} -o m -- "
           "python3 bench.py --workload {workload} --steps 2 --warmup 1 --no-cpu-baseline")


def command(template, directory, workload="cfg2"):
    return template.format(dir=os.path.normpath(directory), workload=workload)


def workload_title(workload):
    sys.path.insert(0, ROOT)
    from ds_splat_amd.synthetic import WORKLOADS
    w = WORKLOADS[workload]
    return "%s: %d Gaussians, %dx%d, SH degree %d, %s" % (w.name, w.n, w.width, w.height, w.sh_degree,
                                                           "forward + backward" if w.backward else "forward")


def short_name(kernel):
    """'void dsx::blend_fwd_kernel<4, true>(...)' -> 'blend_fwd_kernel<4, true>'"""
    name = re.sub(r"^void ", "", kernel).replace("(anonymous namespace)::", "")
    depth, cut = 0, len(name)
    for i, ch in enumerate(name):           # the argument list starts at the first '(' outside <>
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        elif ch == "(" and depth == 0:
            cut = i
            break
    return name[:cut].replace("dsx::", "")


def trace_name(short):
    """The name the library's own event trace (and bench.py's JSON line) uses for a kernel."""
    base = short.split("<")[0]
    if base == "onesweep32_kernel":
        # the depth sort of the Gaussians carries their rectangles through the passes (last template argument;
        # images of more than 255 tiles a side excepted); the tile partition, with 16-bit slots per tile or 32-bit
        # slot words per bin, carries nothing
        return "onesweep32_kernel<sort>" if short.rstrip().endswith("true>") else "onesweep32_kernel<tile partition>"
    return base


def git_commit():
    try:
        head = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True,
                              check=True).stdout.strip()
        status = subprocess.run(["git", "-C", ROOT, "status", "--porcelain", "--untracked-files=no"],
                                capture_output=True, text=True, check=True).stdout.splitlines()
        # (the summaries under profiles/ are this tool's own output, not code that was measured)
        dirty = [line for line in status if not line[3:].startswith("profiles/")]
        return head + ("+uncommitted changes" if dirty else "")
    except Exception:
        return "unknown"


def find_csv(directory, suffix):
    found = sorted(glob.glob(os.path.join(directory, "**", "*" + suffix), recursive=True))
    if not found:
        sys.exit("no *%s under %s" % (suffix, directory))
    return found[-1]


def counters_per_kernel(directory):
    """{short kernel name: {counter: [value per dispatch]}} of a --pmc run"""
    out = collections.defaultdict(lambda: collections.defaultdict(list))
    for r in csv.DictReader(open(find_csv(directory, "counter_collection.csv"))):
        out[short_name(r["Kernel_Name"])][r["Counter_Name"]].append(float(r["Counter_Value"]))
    return out


def kernel_times_ms(directory):
    """{short kernel name: average launch duration in ms} of a --kernel-trace --stats run"""
    return {short_name(r["Name"]): float(r["AverageNs"]) / 1e6
            for r in csv.DictReader(open(find_csv(directory, "kernel_stats.csv")))}


def write(name, lines):
    os.makedirs(PROFILES, exist_ok=True)
    path = os.path.join(PROFILES, name + ".md")
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")
    print("\n".join(lines))
    print("-> " + os.path.relpath(path, ROOT), file=sys.stderr)


def cmd_stats(args):
    rows = list(csv.DictReader(open(find_csv(args.dir, "kernel_stats.csv"))))
    med = collections.defaultdict(list)
    trace = glob.glob(os.path.join(args.dir, "**", "*kernel_trace.csv"), recursive=True)
    if trace:
        for r in csv.DictReader(open(sorted(trace)[-1])):
            med[r["Kernel_Name"]].append(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]))
    lines = ["# Kernel statistics, bench.py (%s)" % workload_title(args.workload), "",
             "Commit: %s" % (args.commit or git_commit()), "",
             "Command (on the MI355X box, repository root, after `export TMPDIR=/tmp`):", "",
             "    " + command(STATS_CMD, args.dir, args.workload), "",
             "rocprofv3 kernel statistics (all launches of the run, warm-up included; the median is taken from the",
             "kernel trace of the same run):", "",
             "| kernel | calls | total ms | avg us | median us | % |", "|---|---|---|---|---|---|"]
    for r in rows:
        m = med.get(r["Name"])
        lines.append("| %s | %s | %.3f | %.1f | %s | %s |" % (
            short_name(r["Name"])[:70], r["Calls"], int(r["TotalDurationNs"]) / 1e6, float(r["AverageNs"]) / 1e3,
            "%.1f" % (statistics.median(m) / 1e3) if m else "-", r["Percentage"]))
    write(args.name, lines)


def algorithmic_bytes(bench):
    """Algorithmic HBM bytes per launch of the HBM-bound kernels, from bench.py's own formulas."""
    sys.path.insert(0, ROOT)
    import bench as bench_module
    cfg = bench["config"]
    m = re.match(r"(\w+): (\d+) Gaussians, (\d+)x(\d+), SH degree (\d+)", cfg["workload"])
    n, w, h, deg = int(m.group(2)), int(m.group(3)), int(m.group(4)), int(m.group(5))
    out = {}
    for k in ("project_fwd_kernel", "gaussian_bwd_kernel", "hist32_kernel", "onesweep32_kernel<sort>",
              "ordered_block_sums_kernel", "emit_ordered_kernel", "onesweep32_kernel<tile partition>"):
        bound, work, _ = bench_module.algorithmic_work(k, n, cfg["num_keys"], w * h, cfg["lists"], (deg + 1) ** 2, None,
                                                       cfg.get("gaussians_with_gradient", 0),
                                                       (w + 15) // 16 <= 255 and (h + 15) // 16 <= 255,
                                                       cfg.get("list_bin_tiles", 1) > 1)
        if bound == "hbm":
            out[k] = work
    return out, n


def cmd_traffic(args):
    fetch = counters_per_kernel(args.fetch_dir)
    wr = counters_per_kernel(args.write_dir)
    bench = json.loads([l for l in open(args.bench_json) if l.startswith("{")][-1])
    copy = "__amd_rocclr_copyBuffer"
    copy_f, copy_w = max(fetch[copy]["FETCH_SIZE"]), max(wr[copy]["WRITE_SIZE"])
    scale_f, scale_w = 1048576.0 / copy_f, 1048576.0 / copy_w
    alg, n = algorithmic_bytes(bench)
    commit = args.commit or git_commit()
    cfg = bench["config"]
    lines = ["# HBM traffic per launch (FETCH_SIZE / WRITE_SIZE), %s" % cfg["workload"], "",
             "Commit: %s" % commit, "",
             "Commands (on the MI355X box, repository root, after `export TMPDIR=/tmp`; one counter per run):", "",
             "    " + command(FETCH_CMD, args.fetch_dir, args.workload),
             "    " + command(WRITE_CMD, args.write_dir, args.workload),
             "    python3 bench_profiles.py traffic %s %s --bench-json <the first run's JSON line> --workload %s --name %s" % (
                 os.path.normpath(args.fetch_dir), os.path.normpath(args.write_dir), args.workload, args.name),
             "",
             "Calibration: `--copy-probe` runs one 1 GiB device-to-device copy (`%s`, reads 1048576 KiB, writes 1048576 KiB)." % copy,
             "The counters read FETCH_SIZE = %.1f KiB and WRITE_SIZE = %.1f KiB for it, so the scale factors are %.4f (fetch) and %.4f (write)." % (
                 copy_f, copy_w, scale_f, scale_w), "",
             "Pairs of the tile lists as built (bins of %d x %d tiles): %d; pairs of per-tile lists: %d; N = %d Gaussians. "
             "Averages over all launches of the run; MB = 1e6 bytes." % (cfg["list_bin_tiles"], cfg["list_bin_tiles"],
                                                                         cfg["num_keys"], cfg["num_keys_per_tile_lists"], n), "",
             "| kernel | launches | FETCH_SIZE KiB (raw) | WRITE_SIZE KiB (raw) | scaled read MB | scaled write MB | scaled total MB | algorithmic MB | traffic / algorithmic |",
             "|---|---|---|---|---|---|---|---|---|"]
    record = {}
    for k in sorted(fetch, key=lambda k: -sum(fetch[k]["FETCH_SIZE"]) - sum(wr.get(k, {}).get("WRITE_SIZE", [0]))):
        if k == copy or k.startswith("stream_probe") or "at::" in k or k.startswith("__amd"):
            continue
        f, w = fetch[k]["FETCH_SIZE"], wr.get(k, {}).get("WRITE_SIZE", [0.0])
        fa, wa = sum(f) / len(f), sum(w) / len(w)
        rb, wb = fa * scale_f * 1024 / 1e6, wa * scale_w * 1024 / 1e6
        tname = trace_name(k)
        tot, cnt = record.get(tname, (0.0, 0))
        record[tname] = (tot + (rb + wb) * 1e6 * len(f), cnt + len(f))      # launch-weighted, per trace name
        a = alg.get(tname)
        lines.append("| %s | %d | %.1f | %.1f | %.1f | %.1f | %.1f | %s | %s |" % (
            k, len(f), fa, wa, rb, wb, rb + wb, "%.1f" % (a / 1e6) if a else "(not HBM-bound)",
            "%.2f" % ((rb + wb) * 1e6 / a) if a else "-"))
    write(args.name, lines)
    path = os.path.join(PROFILES, args.name + ".json")
    with open(path, "w") as f:
        json.dump({"workload": cfg["workload"], "num_keys": cfg["num_keys"], "commit": commit,
                   "scale_fetch": round(scale_f, 4), "scale_write": round(scale_w, 4),
                   "unit": "bytes per launch (FETCH_SIZE + WRITE_SIZE, scaled)",
                   "kernels": {k: int(tot / cnt) for k, (tot, cnt) in record.items()}}, f, indent=1, sort_keys=True)
        f.write("\n")
    print("-> " + os.path.relpath(path, ROOT), file=sys.stderr)


def cmd_sq(args):
    d = counters_per_kernel(args.sq_dir)
    times = kernel_times_ms(args.stats_dir)
    avg = lambda x: sum(x) / len(x)
    lines = ["# SQ counters per kernel (VALU issue, LDS bank conflicts), %s" % workload_title(args.workload), "",
             "Commit: %s" % (args.commit or git_commit()), "",
             "Commands (on the MI355X box, repository root, after `export TMPDIR=/tmp`):", "",
             "    " + command(SQ_CMD, args.sq_dir, args.workload),
             "    " + command(STATS_CMD, args.stats_dir, args.workload) + "    # the `kernel ms` column", "",
             "Averages per launch. A wave64 VALU instruction occupies its SIMD for 4 clocks, so the chip (256 CU x 4 SIMD at 2.4 GHz)",
             "issues at most 614 G wave-instructions/s: `VALU floor` = SQ_INSTS_VALU / 614e9 is the time the kernel's VALU",
             "instructions alone need (quarter-rate instructions such as exp and rcp count once here, so the true floor is higher);",
             "`kernel ms` is the launch average of the kernel-trace run.", "",
             "| kernel | waves | VALU inst / wave | SALU inst / wave | LDS inst / wave | LDS bank-conflict cycles / LDS inst | SQ_INSTS_VALU | VALU floor ms | kernel ms | floor / kernel |",
             "|---|---|---|---|---|---|---|---|---|---|"]
    for k in sorted(d, key=lambda k: -avg(d[k]["SQ_INSTS_VALU"]) if d[k]["SQ_INSTS_VALU"] else 0):
        c = d[k]
        if "at::" in k or k.startswith("__amd") or not c["SQ_WAVES"] or k not in times:
            continue
        waves, valu, salu, lds = avg(c["SQ_WAVES"]), avg(c["SQ_INSTS_VALU"]), avg(c["SQ_INSTS_SALU"]), avg(c["SQ_INSTS_LDS"])
        bank = avg(c["SQ_LDS_BANK_CONFLICT"])
        floor = valu / 614e9 * 1e3
        lines.append("| %s | %d | %d | %d | %d | %.2f | %.3g | %.3f | %.3f | %.0f %% |" % (
            k, waves, valu / waves, salu / waves, lds / waves, bank / max(lds, 1), valu, floor, times[k],
            100 * floor / times[k]))
    write(args.name, lines)


def cmd_mem(args):
    """Vector-memory instructions and atomics per kernel: how many atomic requests the blend backward sends
    (one instruction per blended (tile, entry) with nine active lanes) and what share of its time they are."""
    d = counters_per_kernel(args.mem_dir)
    times = kernel_times_ms(args.stats_dir)
    avg = lambda x: sum(x) / len(x) if x else 0.0
    lines = ["# Vector-memory instructions and L2 atomics per kernel, %s" % workload_title(args.workload), "",
             "Commit: %s" % (args.commit or git_commit()), "",
             "Commands (on the MI355X box, repository root, after `export TMPDIR=/tmp`):", "",
             "    " + command(MEM_CMD, args.mem_dir, args.workload),
             "    " + command(STATS_CMD, args.stats_dir, args.workload) + "    # the `kernel ms` column", "",
             "Averages per launch. `VMEM write inst` counts stores and atomics (the blend backward issues one atomic",
             "instruction per blended (tile, entry), nine lanes active, plus one byte store for the Gaussian's mark, and at",
             "its end the stores of the zeros); `L2 atomic requests` is TCC_ATOMIC summed over the L2 channels.", "",
             "| kernel | waves | VMEM read inst / wave | VMEM write inst / wave | branches / wave | TCP atomic requests | L2 atomic requests | L2 atomics / us | kernel ms |",
             "|---|---|---|---|---|---|---|---|---|"]
    for k in sorted(d, key=lambda k: -avg(d[k]["TCC_ATOMIC_sum"])):
        c = d[k]
        if "at::" in k or k.startswith("__amd") or not c["SQ_WAVES"] or k not in times:
            continue
        waves = avg(c["SQ_WAVES"])
        atom = avg(c["TCC_ATOMIC_sum"])
        lines.append("| %s | %d | %.1f | %.1f | %.1f | %.4g | %.4g | %.0f | %.3f |" % (
            k, waves, avg(c["SQ_INSTS_VMEM_RD"]) / waves, avg(c["SQ_INSTS_VMEM_WR"]) / waves,
            avg(c["SQ_INSTS_BRANCH"]) / waves, avg(c["TCP_TCC_ATOMIC_WITHOUT_RET_REQ_sum"]), atom,
            atom / (times[k] * 1e3), times[k]))
    write(args.name, lines)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    p = sub.add_parser("stats", help="kernel statistics of a --kernel-trace --stats run")
    p.add_argument("dir")
    p.add_argument("--name", required=True)
    p.add_argument("--commit")
    p.set_defaults(fn=cmd_stats)
    p = sub.add_parser("traffic", help="HBM bytes per launch from a FETCH_SIZE run and a WRITE_SIZE run")
    p.add_argument("fetch_dir")
    p.add_argument("write_dir")
    p.add_argument("--bench-json", required=True, help="stdout of one of the two bench.py runs")
    p.add_argument("--name", required=True)
    p.add_argument("--commit")
    p.set_defaults(fn=cmd_traffic)
    p = sub.add_parser("sq", help="instruction counters per kernel from an SQ counter run")
    p.add_argument("sq_dir")
    p.add_argument("stats_dir")
    p.add_argument("--name", required=True)
    p.add_argument("--commit")
    p.set_defaults(fn=cmd_sq)
    p = sub.add_parser("mem", help="vector-memory instructions and atomics per kernel")
    p.add_argument("mem_dir")
    p.add_argument("stats_dir")
    p.add_argument("--name", required=True)
    p.add_argument("--commit")
    p.set_defaults(fn=cmd_mem)
    for p in sub.choices.values():
        p.add_argument("--workload", default="cfg2", help="the bench.py workload the runs were made with")
    args = ap.parse_args()
    args.fn(args)


if __name__ == "__main__":
    main()
