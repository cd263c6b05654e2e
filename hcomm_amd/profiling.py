"""Turn rocprofv3 output into the short tables kept under profiles/.

    python -m hcomm_amd.profiling stats <dir>
        per-kernel duration table (calls, average / min / max ns) from the *_kernel_stats.csv files under <dir>
        (rocprofv3 --kernel-trace --stats --output-format csv -d <dir> -- python3 bench.py ...)

    python -m hcomm_amd.profiling counters <dir>
        mean / min / max counter value per kernel from the *_counter_collection.csv files under <dir>
        (rocprofv3 --pmc FETCH_SIZE --output-format csv -d <dir> -- python3 bench.py ...)

    python -m hcomm_amd.profiling traffic <workload> <lowering> <kernel substring> <fetch dir> <write dir> [source]
        L2 <-> fabric KiB per launch of the kernel whose name contains the substring, written into
        profiles/traffic.json under "<workload>|<lowering>" (bench.py reads it for roofline.traffic).  Both counters
        are scaled by what they read for k_copy in the same runs, whose launches read and write a known size:
        fetch_scale = WRITE_SIZE(k_copy) / FETCH_SIZE(k_copy) (a copy reads what it writes, and WRITE_SIZE counts
        the bytes written one for one; 2.0 when the runs hold no k_copy), write_scale = 1.
"""
import collections
import csv
import glob
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _short(name):
    name = name.replace("(anonymous namespace)::", "")
    return name.split("(")[0] if name.startswith("void ") is False else name[5:].split("(")[0]


def kernel_stats(d):
    rows = []
    for f in glob.glob(os.path.join(d, "**", "*kernel_stats.csv"), recursive=True):
        for r in csv.DictReader(open(f)):
            rows.append((_short(r["Name"]), int(r["Calls"]), float(r["AverageNs"]), float(r["MinNs"]), float(r["MaxNs"])))
    return sorted(rows, key=lambda r: -r[1] * r[2])


def counters(d):
    acc = collections.defaultdict(list)
    for f in glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True):
        for r in csv.DictReader(open(f)):
            acc[(_short(r["Kernel_Name"]), r["Counter_Name"])].append(float(r["Counter_Value"]))
    return {k: (sum(v) / len(v), min(v), max(v), len(v)) for k, v in acc.items()}


def _mean_of(table, substring, counter):
    hits = [(k, v) for k, v in table.items() if substring in k[0] and k[1] == counter]
    if not hits:
        raise SystemExit("no %s rows for a kernel containing %r" % (counter, substring))
    n = sum(v[3] for _, v in hits)
    return sum(v[0] * v[3] for _, v in hits) / n


def main(argv):
    if len(argv) >= 2 and argv[0] == "stats":
        for name, calls, avg, lo, hi in kernel_stats(argv[1]):
            print("| `%s` | %d | %.1f | %.0f | %.0f |" % (name, calls, avg, lo, hi))
    elif len(argv) >= 2 and argv[0] == "counters":
        for (name, ctr), (mean, lo, hi, n) in sorted(counters(argv[1]).items()):
            print("| `%s` | %s | %d | %.1f | %.1f | %.1f |" % (name, ctr, n, mean, lo, hi))
    elif len(argv) >= 6 and argv[0] == "traffic":
        workload, lowering, sub, fdir, wdir = argv[1:6]
        fetch, write = counters(fdir), counters(wdir)
        if any("k_copy" in k[0] for k in fetch):
            scale = round(_mean_of(write, "k_copy", "WRITE_SIZE") / _mean_of(fetch, "k_copy", "FETCH_SIZE"), 4)
            scale_from = "k_copy in the same runs"
        else:  # a workload without copies: the factor every run that has k_copy gives (2.000 +- 0.002)
            scale, scale_from = 2.0, "no k_copy in these runs: the factor of the runs that have one"
        entry = {"kernel": sub, "fetch_kib": round(_mean_of(fetch, sub, "FETCH_SIZE"), 1),
                 "write_kib": round(_mean_of(write, sub, "WRITE_SIZE"), 1),
                 "fetch_scale": scale, "fetch_scale_from": scale_from, "write_scale": 1.0,
                 "source": argv[6] if len(argv) > 6 else ""}
        path = os.path.join(ROOT, "profiles", "traffic.json")
        try:
            doc = json.load(open(path))
        except (OSError, ValueError):
            doc = {"what": "L2 <-> fabric KiB per launch of a workload's dominant kernel (rocprofv3 --pmc FETCH_SIZE / "
                           "WRITE_SIZE); written by python -m hcomm_amd.profiling traffic, read by bench.py",
                   "entries": {}}
        doc["entries"]["%s|%s" % (workload, lowering)] = entry
        json.dump(doc, open(path, "w"), indent=1, sort_keys=True)
        print(json.dumps(entry))
    else:
        raise SystemExit(__doc__)


if __name__ == "__main__":
    main(sys.argv[1:])
