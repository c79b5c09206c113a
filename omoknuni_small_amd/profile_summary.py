"""Turns rocprofv3 CSV output into the short text summaries kept under profiles/.

    python -m omoknuni_small_amd.profile_summary stats  <kernel_trace.csv | kernel_stats.csv> [skip]
    python -m omoknuni_small_amd.profile_summary pmc    <counter_collection.csv> <COUNTER> [copy_bytes [skip]]
    python -m omoknuni_small_amd.profile_summary counters <counter_collection.csv> [skip]
    python -m omoknuni_small_amd.profile_summary traffic <workload> <fetch.csv> <write.csv> <copy_bytes> <out.json> [command [skip]]
    python -m omoknuni_small_amd.profile_summary timeline <workload> [warmup_steps [level ...]]

`stats` prints calls / total / average duration per kernel (and median and minimum, from the trace of the
dispatches).  `pmc` prints, per kernel, the sum of a hardware counter over its dispatches; given the bytes
the calibration copy kernel (k_copy_words) moved each way per launch, it also prints the counter-to-bytes
factor that copy implies and every kernel's traffic in bytes scaled by it.  `counters` prints every counter
of the file per kernel, averaged over its dispatches.  `traffic` writes the scaled FETCH_SIZE and WRITE_SIZE
bytes per launch of the two runs into a JSON file under the workload's name (what bench.py quotes as
roofline.traffic).  `skip` leaves out the first so many dispatches of every selection kernel: with
`bench.py --steps 1 --warmup 0 --seeded-repeats N` the first two are the timed step and its replay, all later
ones the selection on the seeded statistics that bench.py's roofline is quoted on.  `timeline` runs a
benchmark workload on the GPU with the library's timeline records switched on (omk_batch_set_trace): when
every multi-visitor work item of a selection was processed; it prints the chain of crowded nodes of one
steady-state selection: per tree level the node with most visitors, when its wavefront started and ended;
for every level named, all items of that node.
"""
import csv
import sys
from collections import defaultdict


def short(name):
    name = name.replace("omk::", "")
    cut = name.find("(")
    return name[:cut] if cut > 0 else name


def skipped(rows, skip, name_key):
    """rows without the first `skip` dispatches of every selection kernel (in dispatch order): what a
    profile of the selection on the seeded statistics leaves out, the launches of bench.py's timed steps."""
    if not skip:
        return rows
    rows = sorted(rows, key=lambda r: int(r["Dispatch_Id"]))
    seen = defaultdict(set)
    out = []
    for r in rows:
        k = short(r[name_key])
        if "k_select" in k:
            seen[k].add(int(r["Dispatch_Id"]))
            if len(seen[k]) <= skip:
                continue
        out.append(r)
    return out


def stats(path, skip=0):
    rows = list(csv.DictReader(open(path)))
    if rows and "Start_Timestamp" in rows[0]:  # the kernel trace itself: one row per dispatch
        rows = skipped(rows, skip, "Kernel_Name")
        dur = defaultdict(list)
        for r in rows:
            dur[short(r["Kernel_Name"])].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
        total = sum(sum(v) for v in dur.values())
        if skip:
            print("(the first %d dispatches of every selection kernel left out)" % skip)
        print("%-44s %8s %14s %12s %12s %12s %7s" % ("kernel", "calls", "total_us", "avg_us", "median_us", "min_us", "pct"))
        for k in sorted(dur, key=lambda x: -sum(dur[x])):
            v = sorted(dur[k])
            print("%-44s %8d %14.1f %12.2f %12.2f %12.2f %7.2f" % (k[:44], len(v), sum(v), sum(v) / len(v), v[len(v) // 2],
                                                                  v[0], 100.0 * sum(v) / total))
        return
    print("%-44s %8s %14s %12s %7s" % ("kernel", "calls", "total_us", "avg_us", "pct"))
    for r in rows:
        print("%-44s %8d %14.1f %12.2f %7.2f" % (short(r["Name"])[:44], int(r["Calls"]), int(r["TotalDurationNs"]) / 1e3,
                                                  float(r["AverageNs"]) / 1e3, float(r["Percentage"])))


def pmc(path, counter, copy_bytes=None, skip=0):
    rows = skipped(list(csv.DictReader(open(path))), skip, "Kernel_Name")
    if skip:
        print("(the first %d dispatches of every selection kernel left out)" % skip)
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


def counters(path, skip=0):
    rows = skipped(list(csv.DictReader(open(path))), skip, "Kernel_Name")
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


def scaled_bytes(path, counter, copy_bytes, skip=0):
    rows = skipped(list(csv.DictReader(open(path))), skip, "Kernel_Name")
    tot = defaultdict(float)
    calls = defaultdict(int)
    for r in rows:
        if r["Counter_Name"] == counter:
            tot[short(r["Kernel_Name"])] += float(r["Counter_Value"])
            calls[short(r["Kernel_Name"])] += 1
    factor = copy_bytes * calls["k_copy_words"] / tot["k_copy_words"]
    return {k: int(tot[k] / calls[k] * factor) for k in tot if k.startswith("k_") or "k_select" in k}, factor


def traffic(workload, fetch_csv, write_csv, copy_bytes, out_json, command=None, skip=0):
    import json
    import os
    fetch, f_factor = scaled_bytes(fetch_csv, "FETCH_SIZE", copy_bytes, skip)
    write, w_factor = scaled_bytes(write_csv, "WRITE_SIZE", copy_bytes, skip)
    for d in (fetch, write):
        d.pop("k_copy_words", None)
    sel = sum(v for d in (fetch, write) for k, v in d.items() if "k_select" in k)
    doc = json.load(open(out_json)) if os.path.exists(out_json) else {}
    doc[workload] = {
        "note": "HBM bytes per launch: FETCH_SIZE and WRITE_SIZE of two rocprofv3 --pmc runs, each scaled by what the "
                "counter reads for the copy kernel k_copy_words of known size; selection = reset + multi-visitor + "
                "single-visitor kernels of one step",
        "command": command or "bench.py --workload %s" % workload,
        "selection_dispatches_left_out": skip,
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
    print("chain of crowded nodes: per level the node with most visitors (kinds: node = taken as a whole, chain = a node "
          "whose visitors all follow one child, taken by the walk down such nodes, early = published before its visitor "
          "list was complete; a node cut into slices / scatter parts shows their number and the span from the first "
          "start to the last end)")
    print("%5s %9s %9s %7s %9s %9s %8s  %s" % ("level", "node", "visitors", "kind", "start_us", "end_us", "us", "work"))
    names = {0: "node", 1: "slice", 2: "part", 3: "early", 4: "bound", 5: "chain"}
    for d in range(int(depth.max()) + 1):
        at = np.nonzero(depth == d)[0]
        if len(at) == 0:
            continue
        top = at[np.argmax(m[at])]
        same = at[node[at] == node[top]]
        whole = same[(kind[same] == 0) | (kind[same] == 3) | (kind[same] == 5)]
        first = whole[0] if len(whole) else same[0]
        s0, e1 = start[same].min(), end[same].max()
        n_sl, n_pt = int((kind[same] == 1).sum()), int((kind[same] == 2).sum())
        work = "%d slice item(s), %d scatter part(s)" % (n_sl, n_pt) if n_sl or n_pt else ""
        print("%5d %9d %9d %7s %9.1f %9.1f %8.1f  %s" % (d, node[top], m[top], names.get(int(kind[first]), "?"), s0, e1,
                                                       e1 - s0, work))
    # what a slice notes down: time of its thresholds and exact counts, time of its batch(es), entries of its
    # first batch when the thresholds gave it (-1: it searched for the batch itself), visitors it settled
    note = np.stack([(tr[:, 4] & 0xFFFFFFFF), (tr[:, 4] >> 32) & 0xFFFFFFFF, (tr[:, 5] & 0xFFFFFFFF).astype(np.int32),
                     (tr[:, 5] >> 32) & 0xFFFFFFFF], axis=1).astype(np.int64)
    for lv in levels:
        at = np.nonzero(depth == lv)[0]
        top = at[np.argmax(m[at])]
        same = at[node[at] == node[top]]
        same = same[np.argsort(start[same])]
        print("items of node %d at level %d (number = which slice or part of how many; a slice: thr_us = its two "
              "thresholds and the exact counts at them, batch_us = its entries evaluated, ordered, checked and "
              "written, entries = what the thresholds put in its batch, -1 when it had to search for the batch "
              "itself, settled = visitors it settled):" % (node[top], lv))
        print("  %7s %9s %9s %9s %8s %8s %8s %8s %8s" % ("kind", "number", "start_us", "end_us", "us", "thr_us", "batch_us",
                                                    "entries", "settled"))
        for i in same:
            c = int(ctr[i])
            is_slice = int(kind[i]) == 1 or (int(kind[i]) in (0, 3) and len(same) > 1)
            num = "%d/%d" % (c & 0xFFFF, (c >> 16) & 0x3FFF) if int(kind[i]) in (1, 2) else ("0/-" if is_slice else "")
            line = "  %7s %9s %9.1f %9.1f %8.1f" % (names.get(int(kind[i]), "?"), num, start[i], end[i], end[i] - start[i])
            if is_slice:
                line += " %8.1f %8.1f %8d %8d" % (note[i, 0] / 100.0, note[i, 1] / 100.0, note[i, 2], note[i, 3])
            print(line)
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
    print("critical path: the node whose item ended last (%.1f us) and its ancestors (gap_us: from the end of the "
          "node above to this node's start; negative where a child of a heavy node starts before the visitors are "
          "shared out)" % end.max())
    print("%5s %9s %9s %7s %9s %9s %8s %9s" % ("level", "node", "visitors", "kind", "start_us", "end_us", "us", "gap_us"))
    prev_end = 0.0
    for n_at in reversed(chain):
        same = np.nonzero(node == n_at)[0]
        if len(same) == 0:
            continue
        s0, e1 = start[same].min(), end[same].max()
        kinds = set(int(x) for x in kind[same])
        what = "sliced" if 1 in kinds or 2 in kinds else names.get(int(kind[same[0]]), "?")
        print("%5d %9d %9d %7s %9.1f %9.1f %8.1f %9.1f" % (depth[same[0]], n_at, m[same].max(), what, s0, e1, e1 - s0,
                                                        s0 - prev_end))
        prev_end = e1
    by_kind = ", ".join("%s %d" % (names[k], int((kind == k).sum())) for k in sorted(names))
    print("items by kind: %s; visitors per item: median %d, largest %d" % (by_kind, int(np.median(m)), int(m.max())))


if __name__ == "__main__":
    if len(sys.argv) >= 3 and sys.argv[1] == "stats":
        stats(sys.argv[2], int(sys.argv[3]) if len(sys.argv) > 3 else 0)
    elif len(sys.argv) >= 4 and sys.argv[1] == "pmc":
        pmc(sys.argv[2], sys.argv[3], int(sys.argv[4]) if len(sys.argv) > 4 else None, int(sys.argv[5]) if len(sys.argv) > 5 else 0)
    elif len(sys.argv) >= 3 and sys.argv[1] == "counters":
        counters(sys.argv[2], int(sys.argv[3]) if len(sys.argv) > 3 else 0)
    elif len(sys.argv) >= 7 and sys.argv[1] == "traffic":
        traffic(sys.argv[2], sys.argv[3], sys.argv[4], int(sys.argv[5]), sys.argv[6], sys.argv[7] if len(sys.argv) > 7 else None,
                int(sys.argv[8]) if len(sys.argv) > 8 else 0)
    elif len(sys.argv) >= 3 and sys.argv[1] == "timeline":
        timeline(sys.argv[2], int(sys.argv[3]) if len(sys.argv) > 3 else 8, [int(x) for x in sys.argv[4:]])
    else:
        print(__doc__)
        sys.exit(2)
