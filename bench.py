#!/usr/bin/env python3
"""Benchmark of the tree-search hot path on one MI355X.

A step is one pass of the hot path over one batch of concurrent traversals of a seeded
synthetic forest: batched PUCT selection with virtual loss down to the leaves, then the
backup of one value per leaf (update + revert virtual loss, sign flipped per ply), plus
the leaf-key table probes on the workload that has them.  Everything a step touches is
resident in HBM before the timed region starts; nothing returns to the host inside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c0..c4|wide] [--configs c0,c1,...|none]

Prints ONE JSON line.  The top-level fields are those of --workload (default c3, the
"batch 4096" configuration the metric is quoted on); `per_config` holds the same measurement
for every other benchmark configuration (c0 .. c4), each on its own full-size forest.

`value` is traversals per second over whole steps (every traversal is selected AND backed up
inside the timed region; the K timed steps run back to back).  `roofline` prices the selection
against HBM bandwidth with algorithmic bytes (what one selection step has to read: the
statistics of the children that take part, the node header, the legal mask bits, the
virtual-loss update), summed over the K timed steps: after the timed run the statistics are
put back to where they were when it started and the same K steps are run again with the paths
read back after each one.  Durations come from HIP events on the stream the kernels run on.
`parity` compares one more step on the very forest that was timed with the CPU checker (paths,
leaves, N, virtual loss exact; W relative error; near ties as the checker counts them; table
probes).  `cpu_baseline` times the CPU checker on the host cores of the same machine, on a
bounded number of steps of the same workload: the serial array restatement of the reference's
selection / backup loops (one core) and the same arithmetic over the reference's own node
layout (heap nodes, one cache line per atomic field) with its OpenMP loops, at one thread and
at the host's share of cores; `value` is the fastest of them.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
BENCH_CONFIGS = ["c0", "c1", "c2", "c3", "c4"]


class HipEvents:
    """hipEvent timing on a given stream through the HIP runtime the library itself uses."""

    def __init__(self):
        self.hip = C.CDLL("libamdhip64.so")

    def _ok(self, rc, what):
        if rc != 0:
            raise RuntimeError("%s failed with hipError %d" % (what, rc))

    def create(self):
        ev = C.c_void_p()
        self._ok(self.hip.hipEventCreate(C.byref(ev)), "hipEventCreate")
        return ev

    def destroy(self, ev):
        self.hip.hipEventDestroy(ev)

    def record(self, ev, stream):
        self._ok(self.hip.hipEventRecord(ev, C.c_void_p(stream)), "hipEventRecord")

    def elapsed_ms(self, a, b):
        self._ok(self.hip.hipEventSynchronize(b), "hipEventSynchronize")
        ms = C.c_float()
        self._ok(self.hip.hipEventElapsedTime(C.byref(ms), a, b), "hipEventElapsedTime")
        return float(ms.value)

    def device_sync(self):
        self._ok(self.hip.hipDeviceSynchronize(), "hipDeviceSynchronize")


def legal_children_per_node(soa):
    """Number of children of every node that a selection at it has to read."""
    cb, cc = soa["child_begin"].astype(np.int64), soa["child_count"].astype(np.int64)
    n = len(cc)
    if soa.get("legal") is None:
        return cc.copy()
    bits = np.unpackbits(soa["legal"].view(np.uint8), bitorder="little")[:n].astype(np.int64)
    cs = np.concatenate([[0], np.cumsum(bits)])
    return cs[np.minimum(cb + cc, n)] - cs[np.minimum(cb, n)]


class ByteModel:
    """Bytes one step has to move, by the per-unit model:
    selection step at a node with L participating children of F slots:
        L*16 (N, W, P, VL)  [+ L*8 RAVE]  + ceil(F/8) mask bytes (dense slots only)
        + 16 (child range, N_parent, flags) + 8 (virtual-loss update of the chosen child)
    backup of a path node: 24 (N, W, VL read-modify-write), + 4 per leaf value + 4 per path entry."""

    def __init__(self, soa, meta):
        self.L = legal_children_per_node(soa)
        self.cc = soa["child_count"].astype(np.int64)
        self.per_child = 24 if meta.get("has_rave") else 16
        self.pw = bool(meta.get("pw"))
        self.dense = soa.get("legal") is not None

    def step(self, paths, plen, N_at_select):
        n_t, row = paths.shape
        d_idx = np.arange(row)[None, :]
        sel_mask = d_idx < (plen[:, None] - 1)  # a selection happens at every path node but the leaf
        nodes = paths[sel_mask]
        Lsel = self.L[nodes]
        if self.pw:
            k = np.ceil(np.sqrt(np.maximum(N_at_select[nodes].astype(np.float64), 1.0))).astype(np.int64)
            Lsel = np.minimum(Lsel, np.maximum(k, 1))
        mask_bytes = (self.cc[nodes] + 7) // 8 if self.dense else 0
        sel = int((Lsel * self.per_child + mask_bytes + 24).sum()) + int(4 * plen.sum())
        bak = int(24 * plen.sum() + 4 * n_t + 4 * plen.sum())
        return sel, bak, int(sel_mask.sum())


def visits_of(paths, plen, n_nodes):
    """How often every node occurs on the paths of a step (what a backup adds to N)."""
    row = paths.shape[1]
    on_path = np.arange(row)[None, :] < plen[:, None]
    return np.bincount(paths[on_path], minlength=n_nodes).astype(np.int32)


def exact_value_sums(paths, plen, values, n_nodes):
    """What a backup adds to W of every node, in double precision: the leaf of a path takes +value,
    every ply up flips the sign."""
    row = paths.shape[1]
    d_idx = np.arange(row)[None, :]
    on_path = d_idx < plen[:, None]
    sign = np.where(((plen[:, None] - 1 - d_idx) & 1) == 1, -1.0, 1.0)
    contrib = (sign * values.astype(np.float64)[:, None])[on_path]
    return np.bincount(paths[on_path], weights=contrib, minlength=n_nodes)


def cpu_baseline(soa, meta, troots, values, seconds, max_steps):
    """The CPU checker on the host's cores, on a bounded number of steps of the same workload."""
    from oracle import ref_cpu as R
    B, D, vl = len(troots), int(meta["max_depth"]), int(meta["virtual_loss"])
    ref = R.RefTree.from_soa(soa)
    rp = R.make_params(c_puct=meta["c_puct"], virtual_loss=vl, use_rave=bool(meta.get("has_rave")),
                       rave_k=float(meta.get("rave_k", 3000.0)), pw=bool(meta.get("pw")), max_depth=D)
    done = 0
    sel_s = bak_s = 0.0
    t_start = time.perf_counter()
    while done < 2 or (time.perf_counter() - t_start) < seconds / 2:
        a = time.perf_counter()
        rpaths, rlen, rleaf, _ = ref.select_batch(troots, rp, near_ties=False)
        b = time.perf_counter()
        ref.backup_batch(rpaths, rlen, values, vl)
        c = time.perf_counter()
        sel_s += b - a
        bak_s += c - b
        done += 1
        if done >= max_steps:
            break
    del ref
    soa_rate = B * done / (sel_s + bak_s)
    out = {
        "value": soa_rate,
        "unit": "traversals/s",
        "cores": 1,
        "kind": "port",
        "sample": "%d steps of the same workload (same forest, roots and leaf values) through the "
                  "serial CPU restatement of selectChild / applyVirtualLoss / update / revertVirtualLoss" % done,
        "soa_serial_select_traversals_per_s": B * done / sel_s,
        "soa_serial_backups_per_s": B * done / bak_s,
        "soa_serial_traversals_per_s": soa_rate,
        "host_cores_visible": os.cpu_count(),
    }
    # The same arithmetic over the reference's own layout and threading: heap nodes with one
    # cache line per atomic field, shared_ptr child vectors, OpenMP loops with
    # schedule(dynamic, 1).  Timed with one thread and with the host's share of cores; the
    # faster of the three figures becomes `value` (with several threads the traversal
    # order, hence the result, depends on the schedule, as the reference's does).
    if len(soa["N"]) <= 20_000_000:
        from oracle import ref_ptr as RP
        t_build = time.perf_counter()
        pt = RP.PtrTree(soa)
        t_build = time.perf_counter() - t_build
        n_thr = max(1, min(16, os.cpu_count() or 1))
        kw = dict(c_puct=meta["c_puct"], virtual_loss=vl, use_rave=bool(meta.get("has_rave")),
                  rave_k=float(meta.get("rave_k", 3000.0)), pw=bool(meta.get("pw")), max_depth=D)
        rates = {}
        for thr in sorted({1, n_thr}):
            tot, steps_done = 0.0, 0
            t_start = time.perf_counter()
            while steps_done < 2 or (time.perf_counter() - t_start) < seconds / 4:
                _, _, s_s, b_s = pt.step(troots, values, threads=thr, **kw)
                tot += s_s + b_s
                steps_done += 1
                if steps_done >= max_steps:
                    break
            rates[thr] = B * steps_done / tot
        pt.close()
        out["pointer_tree_traversals_per_s"] = {str(k): v for k, v in rates.items()}
        out["pointer_tree_node_bytes"] = RP.PtrTree.node_bytes()
        out["pointer_tree_build_s"] = t_build
        best_thr = max(rates, key=rates.get)
        if rates[best_thr] > soa_rate:
            out["value"] = rates[best_thr]
            out["cores"] = best_thr
            out["sample"] = ("steps of the same workload (same forest, roots and leaf values) through the CPU "
                             "restatement over the reference's node layout (heap nodes, one cache line per "
                             "atomic) and OpenMP loops, %d thread(s); the serial array checker and the "
                             "one-thread figure are given beside it" % best_thr)
    return out


def parity_check(omk, soa, meta, forest, batch, tt, tt_ids, troots, values, params, steps=1):
    """`steps` more steps on the forest that was just timed, on the device and through the CPU checker
    (started from the device's current statistics), compared phase by phase."""
    from oracle import ref_cpu as R
    B, D, vl = len(troots), int(meta["max_depth"]), int(meta["virtual_loss"])
    now = forest.download()
    cur = dict(soa)
    cur.update(N=now["N"], W=now["W"], VL=now["VL"])
    ref = R.RefTree.from_soa(cur)
    rp = R.make_params(c_puct=meta["c_puct"], virtual_loss=vl, use_rave=bool(meta.get("has_rave")),
                       rave_k=float(meta.get("rave_k", 3000.0)), pw=bool(meta.get("pw")), max_depth=D)
    # W: the device adds the values with float atomics in no fixed order, the checker one after the
    # other in binary32 (the reference itself adds from OpenMP threads, in any order); each is
    # compared with the exact sum, |W - exact| / max(|exact|, 1, sqrt(values added to the node)), and
    # with each other
    out = dict(checked_steps=steps, traversals_per_step=B, mismatched_traversals=0, move_lists_equal=True,
               N_equal=True, VL_equal=True, W_max_rel_err=0.0, W_max_rel_err_vs_serial_f32=0.0,
               serial_f32_max_rel_err=0.0, W_max_rel_err_strict=0.0, W_nodes_above_1e5_strict=0,
               near_tie_traversals=0, mismatches_outside_near_ties=0)
    if tt is not None:
        ref_tt = R.RefTT(4)
        ref_tt.log2 = tt.log2
        ref_tt.slots = tt.download()
        out["tt_probes_equal"] = True
        out["tt_hits"] = 0
    for _ in range(steps):
        rpaths, rlen, rleaf, near = ref.select_batch(troots, rp)
        batch.select(params)
        gpaths, glen, gleaf, gact = batch.read()
        bad = (gpaths != rpaths).any(axis=1) | (glen != rlen) | (gleaf != rleaf)
        out["mismatched_traversals"] += int(bad.sum())
        out["mismatches_outside_near_ties"] += int((bad & (near < 0)).sum())
        out["near_tie_traversals"] += int((near >= 0).sum())
        out["move_lists_equal"] &= bool((gact == ref.gather_actions(rpaths, rlen)).all())
        st = forest.download()
        out["VL_equal"] &= bool((st["VL"] == ref.VL).all())
        if tt is not None:
            got = tt.probe_leaves(batch)
            want, hits = ref_tt.probe(soa["hash"][rleaf])
            out["tt_probes_equal"] &= bool((got == want).all())
            out["tt_hits"] += hits
        exact = ref.W.astype(np.float64) + exact_value_sums(rpaths, rlen, values, len(ref.W))
        ref.backup_batch(rpaths, rlen, values, vl)
        batch.backup(vl)
        st = forest.download()
        out["N_equal"] &= bool((st["N"] == ref.N).all())
        out["VL_equal"] &= bool((st["VL"] == ref.VL).all())
        # a node that takes k values in one step passes through partial sums of the size of a random
        # walk of k steps, whatever the order, and binary32 rounds at that size: errors are taken
        # relative to max(|W|, 1, sqrt(k))
        scale = np.maximum(np.maximum(np.abs(exact), 1.0), np.sqrt(visits_of(rpaths, rlen, len(ref.W))))
        gw = st["W"].astype(np.float64)
        out["W_max_rel_err"] = max(out["W_max_rel_err"], float((np.abs(gw - exact) / scale).max()))
        out["serial_f32_max_rel_err"] = max(out["serial_f32_max_rel_err"], float((np.abs(ref.W - exact) / scale).max()))
        out["W_max_rel_err_vs_serial_f32"] = max(out["W_max_rel_err_vs_serial_f32"],
                                                 float((np.abs(gw - ref.W) / scale).max()))
        # the figure as the task words it: device against the serial binary32 checker, relative to max(|W|, 1),
        # no allowance for the number of values a node takes (both sides round differently at the root, which
        # takes every value of the step: see serial_f32_max_rel_err for the checker's own distance from the exact sum)
        strict = np.abs(gw - ref.W) / np.maximum(np.abs(ref.W.astype(np.float64)), 1.0)
        out["W_max_rel_err_strict"] = max(out["W_max_rel_err_strict"], float(strict.max()))
        out["W_nodes_above_1e5_strict"] += int((strict > 1e-5).sum())
        ref.W[:] = st["W"]
    out["ok"] = bool(out["mismatches_outside_near_ties"] == 0 and out["move_lists_equal"] and out["N_equal"]
                     and out["VL_equal"] and out["W_max_rel_err"] <= 1e-5 and out.get("tt_probes_equal", True))
    return out


def traffic_of(workload):
    """HBM bytes per selection from the committed profiler summary (not measured in this run)."""
    tfile = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if not os.path.exists(tfile):
        return None, None
    with open(tfile) as fh:
        tj = json.load(fh)
    if workload not in tj:
        return None, None
    return tj[workload].get("selection_bytes_per_launch"), (
        "profiles/hbm_traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of `%s`, scaled by the 64 MiB copy "
        "kernel; not measured in this run" % tj[workload].get("command", "bench.py --workload %s" % workload))


def measure(omk, synth, name, steps, warmup, seed, cpu_seconds, scale=1.0, parity=True, relaid=False, seeded_repeats=0):
    """Everything bench.py reports about one workload.  relaid: the same forest without the empty
    slots of its board layout (omk_soa_compact_legal), the layout of the reference's own children_
    vectors; everything (byte model, parity, CPU baseline) is then taken on that forest."""
    kw = {}
    if scale != 1.0:
        kw["nodes_per_tree"] = max(1000, int(synth.CONFIGS[name]["nodes_per_tree"] * scale))
    t0 = time.time()
    soa, roots, meta = synth.generate(name, seed=seed, **kw)
    if relaid:
        soa, old_to_new, _ = omk.compact_legal(soa)
        roots = old_to_new[np.asarray(roots)]
        meta = dict(meta, n_nodes=len(soa["N"]))
    gen_s = time.time() - t0
    n_nodes = len(soa["N"])
    B = int(meta["n_traversals"])
    D = int(meta["max_depth"])
    vl = int(meta["virtual_loss"])
    troots = synth.traversal_roots(roots, B)
    values = np.random.default_rng(seed + 1).uniform(-1, 1, B).astype(np.float32)
    params = omk.SelectParams(c_puct=meta["c_puct"], virtual_loss=vl, use_rave=bool(meta.get("has_rave")),
                              rave_k=float(meta.get("rave_k", 3000.0)), pw=bool(meta.get("pw")))

    forest = omk.Forest.from_soa(soa)
    batch = omk.Batch(forest, B, D)
    batch.set_roots(troots)
    batch.set_values(values)
    tt = None
    tt_ids = None
    d_probe = 0
    if meta.get("tt_log2"):
        tt = omk.TranspositionTable(forest, int(meta["tt_log2"]))
        n_ins = 1 << (int(meta["tt_log2"]) - 1)  # 50 % load
        tt_ids = np.unique(np.linspace(0, meta["n_nodes"] - 1, n_ins).astype(np.int64))
        tt.insert(soa["hash"][tt_ids], tt_ids.astype(np.int32))
        d_probe = forest.dev_alloc(B * 4)

    def step():
        batch.select(params)
        if tt is not None:
            tt.probe_leaves_dev(batch, d_probe)
        batch.backup(vl)

    ev = HipEvents()
    stream = forest.get_stream()
    for _ in range(warmup):
        step()
    forest.sync()
    ev.device_sync()
    start = forest.download()  # the statistics the timed steps start from

    K = steps
    e_sel0 = [ev.create() for _ in range(K)]
    e_sel1 = [ev.create() for _ in range(K)]
    e_end = [ev.create() for _ in range(K)]
    t_wall0 = time.perf_counter()
    for i in range(K):
        ev.record(e_sel0[i], stream)
        batch.select(params)
        ev.record(e_sel1[i], stream)
        if tt is not None:
            tt.probe_leaves_dev(batch, d_probe)
        batch.backup(vl)
        ev.record(e_end[i], stream)
    forest.sync()
    ev.device_sync()
    wall_s = time.perf_counter() - t_wall0
    total_ms = ev.elapsed_ms(e_sel0[0], e_end[K - 1])
    sel_step = [ev.elapsed_ms(e_sel0[i], e_sel1[i]) for i in range(K)]
    bak_step = [ev.elapsed_ms(e_sel1[i], e_end[i]) for i in range(K)]
    for e in e_sel0 + e_sel1 + e_end:
        ev.destroy(e)
    sel_ms, bak_ms = sum(sel_step), sum(bak_step)

    # The byte model over the K timed steps: back to the statistics they started from, the same K
    # steps again, the paths read back after each (the value sums of a backup are atomic float adds,
    # so a replayed W can differ from the timed run's in its last bits; the model counts children
    # and path nodes, which that does not move).
    replay = dict(soa)
    replay.update(N=start["N"], W=start["W"], VL=start["VL"])
    forest.upload(replay)
    del replay
    batch.set_roots(troots)
    model = ByteModel(soa, meta)
    N_host = start["N"].copy()
    sel_bytes = bak_bytes = n_sel_steps = 0
    path_nodes = 0
    for i in range(K):
        batch.select(params)
        paths, plen, leaf, _ = batch.read()
        s_b, b_b, n_s = model.step(paths, plen, N_host)
        sel_bytes += s_b
        bak_bytes += b_b
        n_sel_steps += n_s
        path_nodes += int(plen.sum())
        if tt is not None:
            tt.probe_leaves_dev(batch, d_probe)
        batch.backup(vl)
        N_host += visits_of(paths, plen, n_nodes)
    forest.sync()
    end_state = forest.download()
    del start, N_host

    # The selection ON THE SEEDED STATISTICS (the distributions the configuration states: Zipf visit counts,
    # uniform value sums; the K steps above drift away from them with every backup): the seeded statistics are
    # uploaded again and the roots set again before every repeat, outside the events; the byte model is
    # taken on the paths of that very selection.  This is what the roofline is quoted on.
    reps = seeded_repeats if seeded_repeats > 0 else max(3, min(K, 7))
    seeded_ms = []
    e0, e1 = ev.create(), ev.create()
    for _ in range(reps):
        forest.upload(soa)
        batch.set_roots(troots)
        forest.sync()
        ev.record(e0, stream)
        batch.select(params)
        ev.record(e1, stream)
        forest.sync()
        seeded_ms.append(ev.elapsed_ms(e0, e1))
    ev.destroy(e0)
    ev.destroy(e1)
    paths, plen, leaf, _ = batch.read()
    seeded_bytes, _, seeded_steps = model.step(paths, plen, soa["N"])
    seeded_median, seeded_min = float(np.median(seeded_ms)), float(min(seeded_ms))
    del model, paths, plen, leaf
    # back to where the timed steps ended: the parity check below continues from there
    forest.upload(dict(soa, N=end_state["N"], W=end_state["W"], VL=end_state["VL"]))
    batch.set_roots(troots)
    del end_state

    par = parity_check(omk, soa, meta, forest, batch, tt, tt_ids, troots, values, params) if parity else None

    # selection = 1 reset + 1 persistent launch (teams over a work queue of multi-visitor items, and
    # walkers for the lone visitors) when any traversals share a root, else 1 launch of the
    # single-visitor kernel; the roofline is quoted for the kernel that carries the work, with the
    # whole selection phase (HIP events around it on the forest's stream) as its launch duration
    has_groups = len(np.unique(troots)) < B
    # (the library walks a small batch of lone traversals on a wide layout with a legal mask by blocks, one round
    # of 64 child slots per wavefront: the same rule as its launch code)
    fan = int(np.max(soa["child_count"]))
    rounds = 1 if fan <= 64 else 4 if fan <= 256 else 6 if fan <= 384 else 16
    singles = ("k_select_singles_team" if rounds > 1 and soa.get("legal") is not None and B * rounds <= 4096
               else "k_select_singles")
    dominant = "k_select_groups" if has_groups else singles
    sel_ms_step = sel_ms / K
    bak_ms_step = bak_ms / K
    achieved_timed = sel_bytes / (sel_ms * 1e-3) / 1e9
    achieved = seeded_bytes / (seeded_median * 1e-3) / 1e9
    traffic, traffic_source = traffic_of(name) if scale == 1.0 and not relaid else (None, None)
    res = {
        "workload": "%s%s: %d tree(s) x %d nodes, %d traversals per step, depth <= %d, c_puct %.2f, virtual loss %d%s%s%s"
                    % (name, " re-laid without its empty slots (%d nodes kept)" % n_nodes if relaid else "",
                       meta["n_trees"], meta["nodes_per_tree"], B, D, meta["c_puct"], vl,
                       ", RAVE k=%g" % meta["rave_k"] if meta.get("has_rave") else "",
                       ", progressive widening" if meta.get("pw") else "",
                       ", 2^%d-slot table probes" % meta["tt_log2"] if meta.get("tt_log2") else ""),
        "traversals_per_step": B,
        "steps": K,
        "traversals_per_s": B * K / (total_ms * 1e-3),
        "ms_per_step": total_ms / K,
        "select_ms": sel_ms_step,
        "backup_ms": bak_ms_step,
        "select_ms_first_last": [sel_step[0], sel_step[-1]],
        "select_ms_seeded": seeded_median,
        "select_ms_seeded_min": seeded_min,
        "select_traversals_per_s": B / (sel_ms_step * 1e-3),
        "backups_per_s": B / (bak_ms_step * 1e-3),
        "wall_ms_per_step": wall_s * 1e3 / K,
        "mean_path_nodes": path_nodes / float(K * B),
        "selection_steps_per_step": n_sel_steps / float(K),
        "roofline": {
            "bound": "hbm",
            "kernel": dominant,
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "traffic": traffic,
            "traffic_source": traffic_source,
            "algorithmic_bytes": seeded_bytes,
            "algorithmic_bytes_over": "one selection on the seeded statistics of the configuration (uploaded again "
                                      "before every repeat), the paths of that selection read back",
            "launches_per_step": 1,
            "avg_launch_us": seeded_median * 1e3,
            "min_launch_us": seeded_min * 1e3,
            "seeded_repeats": reps,
            "selection_steps": seeded_steps,
            "launch_covers": "the whole selection, HIP events around it on the forest's stream: " +
                             ("k_select_reset + k_select_groups (teams and walkers in one persistent launch)"
                              if has_groups else
                              singles + " alone (no reset launch when every traversal is alone at its root)")
                             + "; rocprofv3's per-kernel averages add up to it",
            # the same figures over the K timed steps, whose statistics drift with every backup (they depend on
            # --steps / --warmup; kept as information)
            "timed_steps": {
                "achieved": achieved_timed,
                "frac": achieved_timed / HBM_PEAK_GBPS,
                "algorithmic_bytes": sel_bytes / float(K),
                "avg_launch_us": sel_ms_step * 1e3,
                "over": "the %d timed steps (replayed from their starting statistics, paths read back after each)" % K,
            },
            "backup_algorithmic_bytes": bak_bytes / float(K),
            "backup_achieved": bak_bytes / (bak_ms * 1e-3) / 1e9,
        },
        "parity": par,
        "generate_s": gen_s,
        "seed": seed,
    }
    if d_probe:
        forest.dev_free(d_probe)
    if tt is not None:
        tt.close()
    batch.close()
    forest.close()
    if cpu_seconds > 0:
        res["cpu_baseline"] = cpu_baseline(soa, meta, troots, values, cpu_seconds, K + warmup)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=BENCH_CONFIGS + ["wide"])
    ap.add_argument("--configs", default=",".join(BENCH_CONFIGS),
                    help="comma-separated workloads measured beside --workload into per_config ('none': only --workload)")
    ap.add_argument("--relaid", default="c2,c4,wide",
                    help="comma-separated board workloads also measured on the forest re-laid without its empty "
                         "slots, into per_config_relaid ('none': skip)")
    ap.add_argument("--head-relaid", action="store_true",
                    help="measure --workload itself on the re-laid forest (for profiler runs of that layout)")
    ap.add_argument("--seed", type=int, default=2025)
    ap.add_argument("--cpu-seconds", type=float, default=12.0,
                    help="budget of the CPU baseline leg of --workload (0 = skip); the other configurations get a third")
    ap.add_argument("--scale", type=float, default=1.0, help="scale nodes_per_tree (debugging only)")
    ap.add_argument("--no-parity", action="store_true", help="skip the comparison with the CPU checker")
    ap.add_argument("--seeded-repeats", type=int, default=0,
                    help="selections timed on the seeded statistics (each after a fresh upload); 0: min(steps, 7), "
                         "at least 3")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MIB",
                    help="only run the plain copy kernel over this many MiB, 10 times (to scale profiler "
                         "traffic counters by) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (independent trees would shard by tree id with no "
              "exchange); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import omoknuni_small_amd as omk
    from omoknuni_small_amd import synth

    if args.copy_calibration > 0:
        nbytes = args.copy_calibration << 20
        f = omk.Forest(16)
        src, dst = f.dev_alloc(nbytes), f.dev_alloc(nbytes)
        f.h2d(src, np.zeros(nbytes // 4, np.uint32))
        for _ in range(10):
            f.dev_copy(dst, src, nbytes)
        f.sync()
        print(json.dumps({"copy_calibration_bytes_each_way": nbytes, "launches": 10}))
        return

    head = measure(omk, synth, args.workload, args.steps, args.warmup, args.seed, args.cpu_seconds, args.scale,
                   parity=not args.no_parity, relaid=args.head_relaid, seeded_repeats=args.seeded_repeats)

    # outside every timed region: three plain copies of 64 MiB, the known-size kernel that a
    # profiler run of this command scales its traffic counters by
    f = omk.Forest(16)
    cal_bytes = 64 << 20
    d_src, d_dst = f.dev_alloc(cal_bytes), f.dev_alloc(cal_bytes)
    for _ in range(3):
        f.dev_copy(d_dst, d_src, cal_bytes)
    f.sync()
    f.dev_free(d_src)
    f.dev_free(d_dst)
    f.close()

    out = {
        "metric": "PUCT traversals/s (selection with virtual loss + value backup per step)",
        "value": head["traversals_per_s"],
        "unit": "traversals/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": head["workload"],
            "traversals_per_step": head["traversals_per_step"],
            "seed": args.seed,
            "mean_path_nodes": head["mean_path_nodes"],
            "selection_steps_per_step": head["selection_steps_per_step"],
        },
        "select_traversals_per_s": head["select_traversals_per_s"],
        "backups_per_s": head["backups_per_s"],
        "select_ms_per_step": head["select_ms"],
        "select_ms_seeded": head["select_ms_seeded"],
        "backup_ms_per_step": head["backup_ms"],
        "wall_ms_per_step": head["wall_ms_per_step"],
        "roofline": head["roofline"],
        "parity": head["parity"],
        "generate_s": head["generate_s"],
    }
    if "cpu_baseline" in head:
        out["cpu_baseline"] = head["cpu_baseline"]

    names = [] if args.configs.strip().lower() in ("", "none") else [c.strip() for c in args.configs.split(",")]
    per = {}
    for name in names:
        if name not in BENCH_CONFIGS + ["wide"]:
            print("bench.py: unknown configuration %r in --configs" % name, file=sys.stderr)
            sys.exit(2)
        if name == args.workload and not args.head_relaid:
            r = head
        else:
            r = measure(omk, synth, name, args.steps, args.warmup, args.seed, args.cpu_seconds / 3.0, args.scale,
                        parity=not args.no_parity, seeded_repeats=args.seeded_repeats)
        per[name] = {
            "workload": r["workload"],
            "select_ms": r["select_ms"],
            "backup_ms": r["backup_ms"],
            "ms_per_step": r["ms_per_step"],
            "traversals_per_s": r["traversals_per_s"],
            "select_traversals_per_s": r["select_traversals_per_s"],
            "backups_per_s": r["backups_per_s"],
            "select_ms_first_last": r["select_ms_first_last"],
            "select_ms_seeded": r["select_ms_seeded"],
            "select_ms_seeded_min": r["select_ms_seeded_min"],
            "roofline": {k: r["roofline"][k] for k in ("kernel", "achieved", "frac", "algorithmic_bytes", "avg_launch_us",
                                                        "timed_steps", "backup_algorithmic_bytes", "backup_achieved",
                                                        "traffic")},
            "parity": r["parity"],
        }
        if "cpu_baseline" in r:
            cb = r["cpu_baseline"]
            per[name]["cpu_baseline"] = {k: cb[k] for k in ("value", "unit", "cores", "kind") if k in cb}
            for k in ("soa_serial_traversals_per_s", "pointer_tree_traversals_per_s"):
                if k in cb:
                    per[name]["cpu_baseline"][k] = cb[k]
    if per:
        out["per_config"] = per
        # a compact copy inside `roofline`: the selection on the seeded statistics of every configuration, and
        # the configuration the target is stated on (c4 in the layout the configuration states, not re-laid)
        brief = {}
        for name, r in per.items():
            rl = r["roofline"]
            brief[name] = {"select_ms": r["select_ms"], "select_ms_seeded": r["select_ms_seeded"],
                           "algorithmic_bytes": rl["algorithmic_bytes"], "achieved": rl["achieved"], "frac": rl["frac"],
                           "traversals_per_s": r["traversals_per_s"],
                           "parity_ok": r["parity"]["ok"] if r["parity"] else None}
            if r["parity"]:
                brief[name]["W_max_rel_err_strict"] = r["parity"]["W_max_rel_err_strict"]
        out["roofline"] = dict(out["roofline"], per_config=brief)
        if "c4" in brief:
            out["roofline"]["north_star"] = dict(brief["c4"], workload=per["c4"]["workload"])

    def short(r):
        d = {
            "workload": r["workload"],
            "select_ms": r["select_ms"],
            "backup_ms": r["backup_ms"],
            "ms_per_step": r["ms_per_step"],
            "traversals_per_s": r["traversals_per_s"],
            "select_traversals_per_s": r["select_traversals_per_s"],
            "backups_per_s": r["backups_per_s"],
            "select_ms_first_last": r["select_ms_first_last"],
            "select_ms_seeded": r["select_ms_seeded"],
            "select_ms_seeded_min": r["select_ms_seeded_min"],
            "roofline": {k: r["roofline"][k] for k in ("kernel", "achieved", "frac", "algorithmic_bytes", "avg_launch_us",
                                                        "timed_steps", "backup_algorithmic_bytes", "backup_achieved",
                                                        "traffic")},
            "parity": r["parity"],
        }
        return d

    relaid = [] if args.relaid.strip().lower() in ("", "none") else [c.strip() for c in args.relaid.split(",")]
    rel = {}
    for name in relaid:
        if name not in BENCH_CONFIGS + ["wide"] or not synth.CONFIGS[name].get("dense"):
            print("bench.py: %r in --relaid is not a board workload" % name, file=sys.stderr)
            sys.exit(2)
        rel[name] = short(measure(omk, synth, name, args.steps, args.warmup, args.seed, 0.0, args.scale,
                                  parity=not args.no_parity, relaid=True, seeded_repeats=args.seeded_repeats))
    if rel:
        out["per_config_relaid"] = rel
    print(json.dumps(out))


if __name__ == "__main__":
    main()
