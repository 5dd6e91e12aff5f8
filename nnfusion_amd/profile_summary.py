"""Text summaries of rocprofv3 runs of bench.py: the tables kept under profiles/.

    python3 -m nnfusion_amd.profile_summary stats    <dir of the --stats run>                      > kernel statistics
    python3 -m nnfusion_amd.profile_summary traffic  <FETCH_SIZE dir> <WRITE_SIZE dir> <probe log>  > HBM bytes per row
    python3 -m nnfusion_amd.profile_summary counters <dir of a --pmc run> <probe log> [row prefix ...]
                                                                                      > counters per row and kernel
    python3 -m nnfusion_amd.profile_summary kernels  <dir of a --pmc run> <last n> [name part ...]
                                                       > counters per kernel: means over its last n dispatches

`bench.py --pmc-probe` launches every configuration row eagerly with a marker launch (probe_read_kernel) ahead of each
and prints the order of the rows as one JSON line ({"pmc_probe": ...}): the probe log is the file that line went to.  The
dispatches between two markers are a row's; their counters are summed over the row's kernels and divided by its launches.
The summaries are written to stdout; each names the command that made its input.
"""
import collections
import csv
import glob
import json
import os
import re
import subprocess
import sys


def demangle(name):
    if name.startswith("_Z"):
        try:
            name = subprocess.run(["c++filt", name], capture_output=True, text=True).stdout.strip() or name
        except OSError:
            pass
    name = name.replace("void ", "").replace("(anonymous namespace)::", "")
    return re.sub(r"\(.*\)$", "", name)


def short(name, width=64):
    """nnf::gemm_sk::kernel<4, 2, ...>(args) -> kernel<4, 2, ...>, cut to `width`."""
    name = demangle(name)
    name = re.sub(r"\b(nnf|gemm_sk)::", "", name)
    # (a name the demangler at hand does not know -- the _Float16 mangling -- : the kernel's name and its literal arguments)
    m = re.match(r"_ZN3nnf\d+([a-z0-9_]+?_kernel)(?:I((?:L[ib]\d+E)+)E)?", name)
    if m:
        args = [("true" if v == "1" else "false") if t == "b" else v for t, v in re.findall(r"L([ib])(\d+)E", m.group(2) or "")]
        name = m.group(1) + (f"<{', '.join(args)}>" if args else "")
    return name[:width]


def csv_rows(directory, suffix):
    files = sorted(glob.glob(os.path.join(directory, "**", "*" + suffix), recursive=True))
    if not files:
        raise SystemExit(f"no *{suffix} under {directory}")
    with open(files[0], newline="") as f:
        return list(csv.DictReader(f))


def probe_order(log):
    with open(log) as f:
        for line in f:
            if line.startswith('{"pmc_probe"'):
                return json.loads(line)["pmc_probe"]
    raise SystemExit("no pmc_probe line in " + log)


def segments(counter_rows, probe):
    """[(row, [dispatch, ...])] with dispatch = {"kernel", "us", counter: value, ...}; and the calibration copies' rows."""
    by_dispatch = collections.OrderedDict()
    for r in sorted(counter_rows, key=lambda r: int(r["Dispatch_Id"])):
        d = by_dispatch.setdefault(int(r["Dispatch_Id"]), {"kernel": r["Kernel_Name"]})
        d[r["Counter_Name"]] = d.get(r["Counter_Name"], 0.0) + float(r["Counter_Value"])
        if r.get("Start_Timestamp") and r.get("End_Timestamp"):
            d["us"] = (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3
    seg, segs, before = None, [], []
    for d in by_dispatch.values():
        if "probe_read_kernel" in d["kernel"]:
            seg = []
            segs.append(seg)
        elif seg is None:
            before.append(d)
        elif "nnf" in d["kernel"]:
            seg.append(d)
    if len(segs) != len(probe["rows"]):
        raise SystemExit(f"{len(segs)} marker launches in the counter file, {len(probe['rows'])} rows in the probe log")
    return list(zip(probe["rows"], segs)), before


def kernels_of(row, dispatches):
    counts = collections.OrderedDict()
    for d in dispatches:
        counts[short(d["kernel"])] = counts.get(short(d["kernel"]), 0) + 1
    return ", ".join(f"{k} x{c // row['launches']}" for k, c in counts.items())


def traffic(fetch_dir, write_dir, log):
    probe = probe_order(log)
    kib = probe["calibration_copy_bytes"] / 1024
    per, scale = {}, {}
    for counter, directory in (("FETCH_SIZE", fetch_dir), ("WRITE_SIZE", write_dir)):
        segs, before = segments(csv_rows(directory, "counter_collection.csv"), probe)
        # the large device-to-device copies among the copy kernels ahead of the first marker (staging copies are small)
        cal = sorted(d.get(counter, 0.0) for d in before if "copyBuffer" in d["kernel"])[-probe["calibration_copies"]:]
        scale[counter] = (kib / (sum(cal) / len(cal)), sum(cal) / len(cal))
        per[counter] = [(row, sum(d.get(counter, 0.0) for d in ds) / row["launches"], kernels_of(row, ds)) for row, ds in segs]
    out = ["rocprofv3 hardware counters: HBM traffic per launch of every benchmark configuration (FETCH_SIZE, WRITE_SIZE)", "",
           "Commands (two runs, one counter each; on the MI355X box, from /tmp with TMPDIR=/tmp):",
           "  rocprofv3 --pmc FETCH_SIZE --kernel-trace --output-format csv -d <FETCH dir> -o fetch -- python3 bench.py --pmc-probe",
           "  rocprofv3 --pmc WRITE_SIZE --kernel-trace --output-format csv -d <WRITE dir> -o write -- python3 bench.py --pmc-probe",
           "  python3 -m nnfusion_amd.profile_summary traffic <FETCH dir> <WRITE dir> <stdout of the first run>", "",
           "bench.py --pmc-probe copies 1 GiB device-to-device four times (the calibration: each copy reads and writes exactly",
           "1048576 KiB), then launches every configuration row eagerly (the decode sweep once per resident layer, the other rows",
           "three times), one marker launch ahead of each row; the counters of a row are those of the dispatches between two",
           "markers, summed over the row's kernels (pre-pass, GEMM or GEMV, second launch) and divided by its launches.", "",
           f"Calibration: FETCH_SIZE reads {scale['FETCH_SIZE'][1]:.1f} KiB for a copy that reads {kib:.0f} KiB: scaled by {scale['FETCH_SIZE'][0]:.3f};",
           f"WRITE_SIZE reads {scale['WRITE_SIZE'][1]:.1f} KiB for {kib:.0f} KiB written: scaled by {scale['WRITE_SIZE'][0]:.3f}.", "",
           f"{'row':<34} {'FETCH KiB':>11} {'WRITE KiB':>10} {'HBM bytes':>12} {'algorithmic':>12} {'ratio':>6}  kernels (dispatches per launch)"]
    machine = []
    for (row, f, ks), (_, w, _) in zip(per["FETCH_SIZE"], per["WRITE_SIZE"]):
        total = int((f * scale["FETCH_SIZE"][0] + w * scale["WRITE_SIZE"][0]) * 1024)
        out.append(f"{row['row']:<34} {f:>11.1f} {w:>10.1f} {total:>12d} {row['algorithmic_bytes']:>12d} "
                   f"{total / row['algorithmic_bytes']:>6.3f}  {ks}")
        machine.append(f"traffic_bytes_per_launch {row['row']} {total}")
    out += ["", "(FETCH / WRITE KiB: raw counter per launch, before scaling.  HBM bytes = FETCH x scale + WRITE x scale.)", "",
            "Machine-readable (bench.py reads these lines, and the kernels column above, at run time):"] + machine
    return out


def stats(directory):
    rows = csv_rows(directory, "kernel_stats.csv")
    out = ["rocprofv3 kernel statistics: bench.py, decode sweep (M=1 fp16 x int4 g128) + the extra configurations", "",
           "Commands (on the MI355X box, from /tmp with TMPDIR=/tmp):",
           "  rocprofv3 --kernel-trace --stats --output-format csv -d <dir> -o bench -- python3 bench.py --no-cpu-baseline",
           "  python3 -m nnfusion_amd.profile_summary stats <dir>", "",
           "Source: bench_kernel_stats.csv (all kernels of the process, parity gate and probes included; durations in ns).", "",
           f"{'kernel':<78} {'calls':>6} {'avg_ns':>10} {'min_ns':>8} {'max_ns':>8} {'pct':>6}"]
    for r in rows:
        if float(r["Percentage"]) >= 0.05:
            out.append(f"{demangle(r['Name'])[:78]:<78} {r['Calls']:>6} {float(r['AverageNs']):>10.0f} {r['MinNs']:>8} {r['MaxNs']:>8} "
                       f"{float(r['Percentage']):>6.2f}")
    return out


def counters(directory, log, prefixes):
    """Per row and kernel: mean duration and mean of every counter of the run, per dispatch; with the derived figures the
    mid-M and M = 4096 summaries quote where their counters are present."""
    probe = probe_order(log)
    segs, _ = segments(csv_rows(directory, "counter_collection.csv"), probe)
    names = sorted({k for _, ds in segs for d in ds for k in d if k not in ("kernel", "us")})
    out = ["counters per dispatch (means over the row's launches; summed over the chip): " + " ".join(names), "",
           f"{'row':<30} {'kernel':<46} {'us':>7} " + " ".join(f"{n[-14:]:>14}" for n in names)]
    derived = []
    for row, ds in segs:
        if prefixes and not any(row["row"].startswith(p) for p in prefixes):
            continue
        by_kernel = collections.OrderedDict()
        for d in ds:
            by_kernel.setdefault(short(d["kernel"], 46), []).append(d)
        for k, group in by_kernel.items():
            mean = {n: sum(d.get(n, 0.0) for d in group) / len(group) for n in names}
            us = sum(d.get("us", 0.0) for d in group) / len(group)
            out.append(f"{row['row'][:30]:<30} {k:<46} {us:>7.1f} " + " ".join(f"{mean[n]:>14.0f}" for n in names))
            extra = []
            if mean.get("TCC_REQ_sum") and "TCC_HIT_sum" in mean:
                extra.append(f"L2 hit {100 * mean['TCC_HIT_sum'] / mean['TCC_REQ_sum']:.1f} %")
            if mean.get("TCC_READ_sum") and us:
                extra.append(f"L2 reads {mean['TCC_READ_sum'] * 128 / us / 1e6:.2f} TB/s")
            if mean.get("SQ_BUSY_CYCLES") and us:
                cyc = mean["SQ_BUSY_CYCLES"] / 32  # per shader engine, 32 of them: the launch in cycles
                extra.append(f"launch {cyc / 1e3:.1f} kcyc at {cyc / us / 1e3:.2f} GHz")
                if "SQ_VALU_MFMA_BUSY_CYCLES" in mean:  # per SIMD, 4 SIMDs x 256 CUs
                    extra.append(f"MFMA busy {100 * mean['SQ_VALU_MFMA_BUSY_CYCLES'] / 1024 / cyc:.1f} %")
            if mean.get("SQ_WAVE_CYCLES"):
                for n, label in (("SQ_ACTIVE_INST_ANY", "instr. active"), ("SQ_WAIT_ANY", "wait (any)"), ("SQ_WAIT_INST_ANY", "wait (instr.)"),
                                 ("SQ_WAIT_INST_LDS", "wait (LDS)")):
                    if n in mean:
                        extra.append(f"{label} {100 * mean[n] / mean['SQ_WAVE_CYCLES']:.1f} %")
            if extra:
                derived.append(f"{row['row'][:30]:<30} {k:<46} " + ", ".join(extra))
    return out + ["", "derived:"] + derived


def kernels(directory, last, parts):
    """Per kernel (no marker launches needed: for `bench.py --gemm-probe`, which launches two kernels some times each): the
    means of duration and counters over the kernel's last `last` dispatches."""
    by_dispatch = collections.OrderedDict()
    for r in sorted(csv_rows(directory, "counter_collection.csv"), key=lambda r: int(r["Dispatch_Id"])):
        d = by_dispatch.setdefault(int(r["Dispatch_Id"]), {"kernel": r["Kernel_Name"]})
        d[r["Counter_Name"]] = d.get(r["Counter_Name"], 0.0) + float(r["Counter_Value"])
        if r.get("Start_Timestamp") and r.get("End_Timestamp"):
            d["us"] = (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3
    groups = collections.OrderedDict()
    for d in by_dispatch.values():
        name = short(d["kernel"], 60)
        if not parts or any(p in name for p in parts):
            groups.setdefault(name, []).append(d)
    names = sorted({k for g in groups.values() for d in g for k in d if k not in ("kernel", "us")})
    out = [f"means over the last {last} dispatches of each kernel; counters summed over the chip", ""]
    for name, g in groups.items():
        g = g[-last:]
        out.append(f"{name}: {len(g)} dispatches, {sum(d.get('us', 0.0) for d in g) / len(g):.1f} us")
        mean = {n: sum(d.get(n, 0.0) for d in g) / len(g) for n in names}
        for n in names:
            out.append(f"    {n:<34} {mean[n]:>16.0f}")
        if mean.get("SQ_BUSY_CYCLES") and mean.get("SQ_VALU_MFMA_BUSY_CYCLES"):
            cyc = mean["SQ_BUSY_CYCLES"] / 32  # per shader engine, 32 of them: the launch in cycles
            us = sum(d.get("us", 0.0) for d in g) / len(g)
            out.append(f"    launch {cyc:.0f} cycles ({cyc / us / 1e3:.2f} GHz); matrix cores busy "
                       f"{100 * mean['SQ_VALU_MFMA_BUSY_CYCLES'] / 1024 / cyc:.1f} % of them (SQ_VALU_MFMA_BUSY_CYCLES is per SIMD, 1024 of them)")
    return out


def main(argv):
    if len(argv) >= 2 and argv[0] == "stats":
        lines = stats(argv[1])
    elif len(argv) == 4 and argv[0] == "traffic":
        lines = traffic(argv[1], argv[2], argv[3])
    elif len(argv) >= 3 and argv[0] == "counters":
        lines = counters(argv[1], argv[2], argv[3:])
    elif len(argv) >= 3 and argv[0] == "kernels":
        lines = kernels(argv[1], int(argv[2]), argv[3:])
    else:
        raise SystemExit(__doc__)
    print("\n".join(lines))


if __name__ == "__main__":
    main(sys.argv[1:])
