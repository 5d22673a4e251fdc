"""Per-kernel, per-grid summary of a rocprofv3 kernel trace (CSV output format).

    python comfyui-int8-fast_amd/profiling/summarise_kernel_trace.py <dir>/<prefix>_kernel_trace.csv

rocprofv3's own --stats table merges every launch of a kernel template; the GEMM kernel runs at
several shapes in one bench.py run, so launches are grouped here by (kernel, workgroups, threads)
and, inside a group, split where the durations fall into clearly separate clusters (a shape with
the same grid but a different K).
"""
import csv
import re
import statistics
import sys


def short(name):
    name = name.replace("i8f::(anonymous namespace)::", "").replace("void ", "")
    name = re.sub(r"\((GemmArgs|MergeArgs, int|SmallMArgs|char const\*.*)\)$", "", name)
    return name[:58]


def clusters(durs, gap=1.35):
    durs = sorted(durs)
    out, cur = [], [durs[0]]
    for d in durs[1:]:
        if d > cur[-1] * gap and len(cur) >= 5:
            out.append(cur)
            cur = [d]
        else:
            cur.append(d)
    out.append(cur)
    return out


def main(path):
    groups = {}
    for r in csv.DictReader(open(path)):
        if "i8f" not in r["Kernel_Name"] and "copyBuffer" not in r["Kernel_Name"]:
            continue
        wg = int(r["Workgroup_Size_X"])
        key = (short(r["Kernel_Name"]), int(r["Grid_Size_X"]) // wg, wg)
        groups.setdefault(key, []).append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    print(f"{'kernel':58s} {'wgs':>6s} {'thr':>4s} {'calls':>6s} {'avg us':>9s} {'median':>9s} {'min':>9s}")
    for (name, wgs, thr), durs in sorted(groups.items(), key=lambda kv: -sum(kv[1])):
        for c in clusters(durs):
            if len(c) < 5:
                continue
            print(f"{name:58s} {wgs:6d} {thr:4d} {len(c):6d} {statistics.fmean(c):9.2f} {statistics.median(c):9.2f} {min(c):9.2f}")


if __name__ == "__main__":
    main(sys.argv[1])
