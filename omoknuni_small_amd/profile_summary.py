"""Turns rocprofv3 CSV output into the short text summaries kept under profiles/.

    python -m omoknuni_small_amd.profile_summary stats  <kernel_stats.csv>
    python -m omoknuni_small_amd.profile_summary pmc    <counter_collection.csv> <COUNTER> [copy_bytes]

`stats` prints calls / total / average duration per kernel.  `pmc` prints, per kernel, the
sum of a hardware counter over its dispatches; given the bytes the calibration copy kernel
(k_copy_words) moved each way per launch, it also prints the counter-to-bytes factor that
copy implies and every kernel's traffic in bytes scaled by it.
"""
import csv
import sys
from collections import defaultdict


def short(name):
    name = name.replace("omk::", "")
    cut = name.find("(")
    return name[:cut] if cut > 0 else name


def stats(path):
    rows = list(csv.DictReader(open(path)))
    print("%-44s %8s %14s %12s %7s" % ("kernel", "calls", "total_us", "avg_us", "pct"))
    for r in rows:
        print("%-44s %8d %14.1f %12.2f %7.2f" % (short(r["Name"])[:44], int(r["Calls"]), int(r["TotalDurationNs"]) / 1e3,
                                                  float(r["AverageNs"]) / 1e3, float(r["Percentage"])))


def pmc(path, counter, copy_bytes=None):
    rows = list(csv.DictReader(open(path)))
    tot = defaultdict(float)
    calls = defaultdict(int)
    for r in rows:
        if r["Counter_Name"] != counter:
            continue
        k = short(r["Kernel_Name"])
        tot[k] += float(r["Counter_Value"])
        calls[k] += 1
    factor = None
    if copy_bytes and calls.get("k_copy_words"):
        factor = copy_bytes * calls["k_copy_words"] / tot["k_copy_words"]
        print("calibration: k_copy_words moved %d bytes per launch, %s read %.1f per launch -> %.2f bytes per count"
              % (copy_bytes, counter, tot["k_copy_words"] / calls["k_copy_words"], factor))
    print("%-44s %8s %16s %16s %s" % ("kernel", "calls", counter + "_sum", "per_call", "bytes_per_call" if factor else ""))
    for k in sorted(tot, key=lambda x: -tot[x]):
        line = "%-44s %8d %16.1f %16.1f" % (k[:44], calls[k], tot[k], tot[k] / calls[k])
        if factor:
            line += " %16.0f" % (tot[k] / calls[k] * factor)
        print(line)


if __name__ == "__main__":
    if len(sys.argv) >= 3 and sys.argv[1] == "stats":
        stats(sys.argv[2])
    elif len(sys.argv) >= 4 and sys.argv[1] == "pmc":
        pmc(sys.argv[2], sys.argv[3], int(sys.argv[4]) if len(sys.argv) > 4 else None)
    else:
        print(__doc__)
        sys.exit(2)
