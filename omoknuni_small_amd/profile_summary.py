"""Turns rocprofv3 CSV output into the short text summaries kept under profiles/.

    python -m omoknuni_small_amd.profile_summary stats  <kernel_stats.csv>
    python -m omoknuni_small_amd.profile_summary pmc    <counter_collection.csv> <COUNTER> [copy_bytes]
    python -m omoknuni_small_amd.profile_summary counters <counter_collection.csv>
    python -m omoknuni_small_amd.profile_summary traffic <workload> <fetch.csv> <write.csv> <copy_bytes> <out.json> [command]
    OMK_FOREST_LIB=omoknuni_small_amd/libomk_forest_trace.so \
    python -m omoknuni_small_amd.profile_summary timeline <workload> [warmup_steps [level ...]]

`stats` prints calls / total / average duration per kernel.  `pmc` prints, per kernel, the
sum of a hardware counter over its dispatches; given the bytes the calibration copy kernel
(k_copy_words) moved each way per launch, it also prints the counter-to-bytes factor that
copy implies and every kernel's traffic in bytes scaled by it.  `counters` prints every counter of
the file per kernel, averaged over its dispatches.  `traffic` writes the scaled FETCH_SIZE and
WRITE_SIZE bytes per launch of the two runs into a JSON file under the workload's name (what
bench.py quotes as roofline.traffic).  `timeline` runs a benchmark
workload on the GPU through the measurement build of the library (make -C csrc trace), which records
when every multi-visitor work item of a selection was processed, and prints the chain of crowded
nodes of one steady-state selection: per tree level the node with most visitors, when its wavefront
started and ended, and what it did; for every level named, all items of that node.
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


def counters(path):
    rows = list(csv.DictReader(open(path)))
    tot = defaultdict(lambda: defaultdict(float))
    calls = defaultdict(lambda: defaultdict(int))
    names = []
    for r in rows:
        k, c = short(r["Kernel_Name"]), r["Counter_Name"]
        if c not in names:
            names.append(c)
        tot[k][c] += float(r["Counter_Value"])
        calls[k][c] += 1
    print("per dispatch, averaged over the kernel's dispatches")
    print("%-44s %8s " % ("kernel", "calls") + " ".join("%20s" % c for c in names))
    first = names[0]
    for k in sorted(tot, key=lambda x: -tot[x][first]):
        print("%-44s %8d " % (k[:44], calls[k][first]) + " ".join("%20.1f" % (tot[k][c] / max(1, calls[k][c])) for c in names))


def scaled_bytes(path, counter, copy_bytes):
    rows = list(csv.DictReader(open(path)))
    tot = defaultdict(float)
    calls = defaultdict(int)
    for r in rows:
        if r["Counter_Name"] == counter:
            tot[short(r["Kernel_Name"])] += float(r["Counter_Value"])
            calls[short(r["Kernel_Name"])] += 1
    factor = copy_bytes * calls["k_copy_words"] / tot["k_copy_words"]
    return {k: int(tot[k] / calls[k] * factor) for k in tot if k.startswith("k_") or "k_select" in k}, factor


def traffic(workload, fetch_csv, write_csv, copy_bytes, out_json, command=None):
    import json
    import os
    fetch, f_factor = scaled_bytes(fetch_csv, "FETCH_SIZE", copy_bytes)
    write, w_factor = scaled_bytes(write_csv, "WRITE_SIZE", copy_bytes)
    for d in (fetch, write):
        d.pop("k_copy_words", None)
    sel = sum(v for d in (fetch, write) for k, v in d.items() if "k_select" in k)
    doc = json.load(open(out_json)) if os.path.exists(out_json) else {}
    doc[workload] = {
        "note": "HBM bytes per launch: FETCH_SIZE and WRITE_SIZE of two rocprofv3 --pmc runs, each scaled by what the "
                "counter reads for the copy kernel k_copy_words of known size; selection = reset + multi-visitor + "
                "single-visitor kernels of one step",
        "command": command or "bench.py --workload %s" % workload,
        "bytes_per_count": {"FETCH_SIZE": round(f_factor, 2), "WRITE_SIZE": round(w_factor, 2)},
        "fetch_bytes": fetch, "write_bytes": write, "selection_bytes_per_launch": sel}
    with open(out_json, "w") as fh:
        json.dump(doc, fh, indent=1, sort_keys=True)
    print("%s: selection moves %d bytes per launch (fetch + write of its kernels)" % (workload, sel))


def timeline(workload, warmup=8, levels=()):
    import numpy as np
    import omoknuni_small_amd as omk
    from omoknuni_small_amd import synth

    soa, roots, meta = synth.generate(workload, seed=2025)
    B, D, vl = int(meta["n_traversals"]), int(meta["max_depth"]), int(meta["virtual_loss"])
    troots = synth.traversal_roots(roots, B)
    values = np.random.default_rng(2026).uniform(-1, 1, B).astype(np.float32)
    sp = omk.SelectParams(c_puct=meta["c_puct"], virtual_loss=vl, use_rave=bool(meta.get("has_rave")),
                          rave_k=float(meta.get("rave_k", 3000.0)), pw=bool(meta.get("pw")))
    forest = omk.Forest.from_soa(soa)
    batch = omk.Batch(forest, B, D)
    batch.set_roots(troots)
    batch.set_values(values)
    for _ in range(int(warmup)):
        batch.select(sp)
        batch.backup(vl)
    batch.enable_trace()
    batch.select(sp)
    tr = batch.debug_trace()
    batch.enable_trace(False)
    batch.read()  # reports a selection that was given up (and reuses the staging memory the records were in)
    batch.backup(vl)
    t0 = tr[:, 0].min()
    start = (tr[:, 0] - t0) / 100.0  # microseconds
    end = (tr[:, 1] - t0) / 100.0
    m = (tr[:, 2] & 0xFFFFFFFF).astype(np.int64)
    depth = ((tr[:, 2] >> 32) & 0xFFFFFFF).astype(np.int64)
    kind = ((tr[:, 2] >> 60) & 7).astype(np.int64)
    node = (tr[:, 3] & 0xFFFFFFFF).astype(np.int64)
    ctr = (tr[:, 3] >> 32) & 0xFFFFFFFF
    walks = kind == 6  # lone visitors walked by the walker blocks of the persistent launch
    w_start, w_end, w_depth = start[walks], end[walks], depth[walks]
    span_all = end.max()
    keep = ~walks
    tr, start, end, m, depth, kind, node, ctr = tr[keep], start[keep], end[keep], m[keep], depth[keep], kind[keep], node[keep], ctr[keep]
    print("workload %s, selection number %d: %d multi-visitor items traced, span %.1f us (100 MHz clock)"
          % (workload, int(warmup) + 1, len(tr), end.max()))
    if len(w_end):
        dur = w_end - w_start
        print("lone visitors walked inside the persistent launch: %d walks, first start %.1f us, last end %.1f us "
              "(median walk %.1f us, longest %.1f us, median start depth %d); everything ended at %.1f us"
              % (len(w_end), w_start.min(), w_end.max(), float(np.median(dur)), dur.max(), int(np.median(w_depth)), span_all))
    print("chain of crowded nodes: per level the node with most visitors (kinds: node = taken as a whole, chain = a node whose visitors all follow one child, taken by the walk down such nodes, "
          "early = published before its visitor list was complete; a node cut into slices / scatter parts shows "
          "their number and the span from the first start to the last end)")
    ph = np.stack([(tr[:, 4 + q // 2] >> (32 * (q % 2))) & 0xFFFFFFFF for q in range(16)], axis=1) / 100.0
    print("phase columns (us of the owner wavefront, summed over the node's items): load = children loaded and "
          "scored, thr = threshold search and exact counts, ord = entries evaluated and put in order, emit = "
          "emission and checks, settle = all of the settling (includes thr, ord, emit), part = partition or its "
          "hand-over; parts of thr (and of the thresholds a slice derives): probe = run probe, act = bounds and "
          "active children, srch = threshold search, cnt = exact counts; 1win = the one-winner check; runL / runW = length search and emission of runs of one child; "
          "mrg = the direct merge of a node where one child wins nearly every time (or the failed attempt at it)")
    print("%5s %9s %9s %7s %9s %9s %8s %6s %6s %6s %6s %6s %6s | %5s %5s %5s %5s %5s %5s %5s %5s  %s" % (
        "level", "node", "visitors", "kind", "start_us", "end_us", "us", "load", "thr", "ord", "emit", "settle", "part",
        "probe", "act", "srch", "cnt", "1win", "runL", "runW", "mrg", "work"))
    names = {0: "node", 1: "slice", 2: "part", 3: "early", 4: "job", 5: "chain"}
    for d in range(int(depth.max()) + 1):
        at = np.nonzero(depth == d)[0]
        if len(at) == 0:
            continue
        top = at[np.argmax(m[at])]
        same = at[node[at] == node[top]]
        whole = same[(kind[same] == 0) | (kind[same] == 3) | (kind[same] == 5)]
        jobs = same[kind[same] == 4]
        first = whole[0] if len(whole) else same[0]
        s0, e1 = start[same].min(), end[same].max()
        n_sl, n_pt = int((kind[same] == 1).sum()), int((kind[same] == 2).sum())
        batches = int(sum(int(c) & 0xFF for c in ctr[same]))
        runs = int(sum((int(c) >> 8) & 0xFF for c in ctr[same]))
        work = "%d batch(es), %d run(s)" % (batches, runs)
        if n_sl or n_pt:
            work += ", %d slice item(s), %d scatter part(s)" % (n_sl, n_pt)
        if len(jobs):
            work += ", order and partition as a job %.1f-%.1f" % (start[jobs].min(), end[jobs].max())
            same = same[kind[same] != 4]
            s0, e1 = start[same].min(), end[same].max()
        p = ph[same].sum(axis=0)
        print("%5d %9d %9d %7s %9.1f %9.1f %8.1f %6.1f %6.1f %6.1f %6.1f %6.1f %6.1f | %5.1f %5.1f %5.1f %5.1f %5.1f %5.1f %5.1f %5.1f  %s" % (
            d, node[top], m[top], names.get(int(kind[first]), "?"), s0, e1, e1 - s0, p[4], p[0], p[2], p[3], p[5], p[6],
            p[8], p[9], p[10], p[11], p[12], p[13], p[14], p[15], work))
    for lv in levels:
        at = np.nonzero(depth == lv)[0]
        top = at[np.argmax(m[at])]
        same = at[node[at] == node[top]]
        same = same[np.argsort(start[same])]
        print("items of node %d at level %d (slice / part number of a heavy node in `work`):" % (node[top], lv))
        for i in same:
            c = int(ctr[i])
            print("  %7s %9.1f %9.1f %8.1f %6.1f %6.1f %6.1f %6.1f %6.1f %6.1f | %5.1f %5.1f %5.1f %5.1f %5.1f %5.1f %5.1f %5.1f  %d batch(es), %d run(s), last batch %d entries"
                  % (names.get(int(kind[i]), "?"), start[i], end[i], end[i] - start[i], ph[i, 4], ph[i, 0], ph[i, 2], ph[i, 3],
                     ph[i, 5], ph[i, 6], ph[i, 8], ph[i, 9], ph[i, 10], ph[i, 11], ph[i, 12], ph[i, 13], ph[i, 14], ph[i, 15], c & 0xFF, (c >> 8) & 0xFF, c >> 16))
    # the critical path: the item that ended last, and the nodes above it up to the root
    cb, cc = soa["child_begin"].astype(np.int64), soa["child_count"].astype(np.int64)
    parent = np.full(len(cb), -1, np.int64)
    has = np.nonzero(cc > 0)[0]
    parent[np.repeat(cb[has], cc[has]) + (np.arange(int(cc[has].sum())) - np.repeat(np.cumsum(cc[has]) - cc[has], cc[has]))] = \
        np.repeat(has, cc[has])
    chain = []
    n_at = int(node[np.argmax(end)])
    while n_at >= 0:
        chain.append(n_at)
        n_at = int(parent[n_at])
    print("critical path: the node whose item ended last (%.1f us) and its ancestors" % end.max())
    print("(mrg = the direct merge or the attempt at it: m.list = the dominant child chosen, its entries evaluated and "
          "checked; m.rank = counts and ranks of the other children's entries, or, times 1 us, why the merge was "
          "refused: 1 too many children in question, 2 too many entries by the estimate, 3 too many entries, 5 the "
          "dominant child's scores rise, 4x / 6-9 a check failed; the rest of mrg is writing the order)")
    print("%5s %9s %9s %9s %9s %8s %9s | %6s %6s %6s %6s %6s %6s %6s %6s %6s %6s" % (
        "level", "node", "visitors", "start_us", "end_us", "us", "gap_us", "load", "1win", "mrg", "m.list", "m.rank",
        "thr", "ord", "emit", "settle", "part"))
    prev_end = 0.0
    for n_at in reversed(chain):
        same = np.nonzero(node == n_at)[0]
        if len(same) == 0:
            continue
        s0, e1 = start[same].min(), end[same].max()
        p = ph[same].sum(axis=0)
        print("%5d %9d %9d %9.1f %9.1f %8.1f %9.1f | %6.1f %6.1f %6.1f %6.1f %6.1f %6.1f %6.1f %6.1f %6.1f %6.1f" % (
            depth[same[0]], n_at, m[same].max(), s0, e1, e1 - s0, s0 - prev_end, p[4], p[12], p[15], p[7], p[1],
            p[0], p[2], p[3], p[5], p[6]))
        prev_end = e1
    by_kind = ", ".join("%s %d" % (names[k], int((kind == k).sum())) for k in sorted(names))
    print("items by kind: %s; visitors per item: median %d, largest %d" % (by_kind, int(np.median(m)), int(m.max())))


if __name__ == "__main__":
    if len(sys.argv) >= 3 and sys.argv[1] == "stats":
        stats(sys.argv[2])
    elif len(sys.argv) >= 4 and sys.argv[1] == "pmc":
        pmc(sys.argv[2], sys.argv[3], int(sys.argv[4]) if len(sys.argv) > 4 else None)
    elif len(sys.argv) >= 3 and sys.argv[1] == "counters":
        counters(sys.argv[2])
    elif len(sys.argv) >= 7 and sys.argv[1] == "traffic":
        traffic(sys.argv[2], sys.argv[3], sys.argv[4], int(sys.argv[5]), sys.argv[6], sys.argv[7] if len(sys.argv) > 7 else None)
    elif len(sys.argv) >= 3 and sys.argv[1] == "timeline":
        timeline(sys.argv[2], int(sys.argv[3]) if len(sys.argv) > 3 else 8, [int(x) for x in sys.argv[4:]])
    else:
        print(__doc__)
        sys.exit(2)
