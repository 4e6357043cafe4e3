"""Condenses rocprofv3 CSV output of bench.py runs into the short text kept under profiles/.

    python3 -m fyusenet_amd.rocprof_summary --dir D --name N [--kernel REGEX] [--bench-json FILE --kind plain|residual --traffic-out profiles/hbm_traffic.txt]

Expects, under D, what these commands leave (N names the workload run, `copy` the calibration run):
    rocprofv3 --kernel-trace --stats --output-format csv -d D/trace -o N    -- python3 bench.py --workload ...
    rocprofv3 --pmc FETCH_SIZE --kernel-trace --output-format csv -d D/fetch -o N    -- python3 bench.py --workload ...
    rocprofv3 --pmc WRITE_SIZE --kernel-trace --output-format csv -d D/write -o N    -- python3 bench.py --workload ...
    rocprofv3 --pmc FETCH_SIZE --kernel-trace --output-format csv -d D/fetch -o copy -- python3 bench.py --workload copy ...
    rocprofv3 --pmc WRITE_SIZE --kernel-trace --output-format csv -d D/write -o copy -- python3 bench.py --workload copy ...
The copy workload moves 64 x 1024 x 1024 fp32 (262144 KiB) each way per launch; what FETCH_SIZE / WRITE_SIZE read for it
gives the factor that turns the counters into bytes.  With --bench-json (bench.py's JSON line of the same workload, whose
roofline.kernel string is the key) a line `kind <TAB> fetch bytes <TAB> write bytes <TAB> kernel` is appended to the
traffic table that bench.py reads for roofline.traffic.
"""
import argparse
import csv
import glob
import json
import os
import re

COPY_KIB = 262144.0


def _find(d, name, suffix):
    hits = glob.glob(os.path.join(d, "**", "%s_%s.csv" % (name, suffix)), recursive=True)
    return hits[0] if hits else None


def stats_table(path, top=12):
    rows = list(csv.DictReader(open(path)))
    out = []
    for r in rows[:top]:
        out.append("%-100s calls=%-6s avg_us=%9.2f pct=%6s" % (r["Name"][:100], r["Calls"], float(r["AverageNs"]) / 1e3, r["Percentage"]))
    return out


def trace_durations(path, regex):
    rx = re.compile(regex)
    d = {}
    for r in csv.DictReader(open(path)):
        if rx.search(r["Kernel_Name"]):
            d.setdefault(r["Kernel_Name"], []).append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    return d


def counter_avg(path, counter, regex):
    rx = re.compile(regex)
    v = {}
    for r in csv.DictReader(open(path)):
        if r["Counter_Name"] == counter and rx.search(r["Kernel_Name"]):
            v.setdefault(r["Kernel_Name"], []).append(float(r["Counter_Value"]))
    return {k: (sum(x) / len(x), len(x)) for k, x in v.items()}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--dir", required=True)
    ap.add_argument("--name", required=True)
    ap.add_argument("--kernel", default="conv_mfma|conv_p16|conv_kr16|conv_d16|conv_e16dw|conv_h16|conv_rows|conv3x3|dwconv|gemv|pool|reduce")
    ap.add_argument("--bench-json")
    ap.add_argument("--kind", default="plain")
    ap.add_argument("--traffic-out")
    a = ap.parse_args()
    st = _find(os.path.join(a.dir, "trace"), a.name, "kernel_stats")
    if st:
        print("== kernel stats (--stats)")
        print("\n".join(stats_table(st)))
    tr = _find(os.path.join(a.dir, "trace"), a.name, "kernel_trace")
    if tr:
        print("== kernel trace, launches matching /%s/" % a.kernel)
        for k, d in sorted(trace_durations(tr, a.kernel).items(), key=lambda kv: -sum(kv[1])):
            d = sorted(d)
            print("%-100s n=%-6d avg_us=%8.2f median=%8.2f min=%8.2f" % (k[:100], len(d), sum(d) / len(d), d[len(d) // 2], d[0]))
    bytes_by_kernel = {}
    for counter, sub in (("FETCH_SIZE", "fetch"), ("WRITE_SIZE", "write")):
        f = _find(os.path.join(a.dir, sub), a.name, "counter_collection")
        c = _find(os.path.join(a.dir, sub), "copy", "counter_collection")
        if not f or not c:
            continue
        cal = counter_avg(c, counter, "concat")
        if not cal:
            continue
        cal_v = list(cal.values())[0][0]
        factor = COPY_KIB / cal_v
        print("== %s: copy kernel reads %.1f for %.0f KiB moved -> factor %.4f" % (counter, cal_v, COPY_KIB, factor))
        for k, (v, n) in sorted(counter_avg(f, counter, a.kernel).items(), key=lambda kv: -kv[1][0]):
            mb = v * factor * 1024 / 1e6
            print("%-100s n=%-6d avg=%10.1f -> %8.2f MB per launch" % (k[:100], n, v, mb))
            bytes_by_kernel.setdefault(k, {})[sub] = v * factor * 1024
    if a.bench_json and a.traffic_out and bytes_by_kernel:
        rec = json.loads(open(a.bench_json).read().strip().splitlines()[-1])
        info = rec["roofline"]["kernel"]
        # the workload's dominant kernel = the matching kernel with the most bytes
        k, b = max(bytes_by_kernel.items(), key=lambda kv: sum(kv[1].values()))
        if "fetch" in b and "write" in b:
            with open(a.traffic_out, "a") as f:
                f.write("%s\t%.0f\t%.0f\t%s\n" % (a.kind, b["fetch"], b["write"], info))
            print("== traffic table: %s  fetch %.2f MB  write %.2f MB  [%s]" % (a.kind, b["fetch"] / 1e6, b["write"] / 1e6, info))


if __name__ == "__main__":
    main()
