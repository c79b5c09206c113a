"""Seeded synthetic forests of the benchmark configurations (host side, numpy arrays).

The generator itself is csrc/omk_synth.cpp (libomk_synth.so); this module names the five
workloads, scales them, and returns the arrays in the layout Forest.upload() takes.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


class _Desc(C.Structure):
    _fields_ = [("n_trees", C.c_int64), ("nodes_per_tree", C.c_int64), ("dense", C.c_int32), ("fanout", C.c_int32),
                ("legal_frac", C.c_double), ("last_legal", C.c_int32), ("poisson_lambda", C.c_double),
                ("fan_min", C.c_int32), ("fan_max", C.c_int32), ("zipf_s", C.c_double), ("n_cap", C.c_int32),
                ("logit_sigma", C.c_double), ("max_depth", C.c_int32), ("growth_width", C.c_int32),
                ("has_rave", C.c_int32), ("sort_by_prior", C.c_int32), ("pw", C.c_int32), ("with_hash", C.c_int32),
                ("c_puct", C.c_float), ("virtual_loss", C.c_int32), ("seed", C.c_uint64)]


class _Out(C.Structure):
    _fields_ = [(k, C.c_void_p) for k in ("N", "W", "P", "VL", "rN", "rW", "child_begin", "child_count", "action",
                                          "legal", "hash", "depth", "roots", "used")]


# The five workloads.  n_traversals is the number of concurrent root-to-leaf descents of one
# step; traversal t starts at the root of tree t % n_trees.
CONFIGS = {
    # Gomoku 15x15, one tree: 225 slots per expanded node, about half of the cells occupied
    "c0": dict(n_trees=1, nodes_per_tree=200_000, dense=1, fanout=225, legal_frac=0.5, last_legal=0, zipf_s=1.2,
               n_cap=10_000, logit_sigma=1.0, max_depth=12, growth_width=64, n_traversals=64, c_puct=1.4,
               virtual_loss=3),
    # Gomoku 15x15 leaf-parallel self-play: 256 independent trees, one descent per tree and step
    "c1": dict(n_trees=256, nodes_per_tree=50_000, dense=1, fanout=225, legal_frac=0.5, last_legal=0, zipf_s=1.2,
               n_cap=10_000, logit_sigma=1.0, max_depth=12, growth_width=16, n_traversals=256, c_puct=1.4,
               virtual_loss=3),
    # Go 19x19: 361 points + pass, about 40 % occupied; 64 trees, 16 descents per tree
    "c2": dict(n_trees=64, nodes_per_tree=1_000_000, dense=1, fanout=362, legal_frac=0.6, last_legal=1, zipf_s=1.1,
               n_cap=10_000, logit_sigma=1.5, max_depth=30, growth_width=16, n_traversals=1024, c_puct=1.4,
               virtual_loss=3),
    # chess-like variable fan-out, children stored by descending prior, progressive widening
    "c3": dict(n_trees=1, nodes_per_tree=4_000_000, dense=0, poisson_lambda=35.0, fan_min=1, fan_max=218,
               zipf_s=1.2, n_cap=10_000, logit_sigma=1.0, max_depth=24, growth_width=4096, sort_by_prior=1, pw=1,
               n_traversals=4096, c_puct=1.4, virtual_loss=3),
    # Go 19x19 stress: one 16M-node tree with RAVE statistics and position keys for table probes
    "c4": dict(n_trees=1, nodes_per_tree=16_000_000, dense=1, fanout=362, legal_frac=0.6, last_legal=1, zipf_s=1.1,
               n_cap=10_000, logit_sigma=1.5, max_depth=30, growth_width=2048, has_rave=1, with_hash=1,
               n_traversals=16384, c_puct=1.4, virtual_loss=3, rave_k=1000.0, tt_log2=24),
    # Not one of the benchmark configurations: a wide forest in which every descent is alone in
    # its tree, the regime where selection is bound by HBM bandwidth rather than by the chain of
    # crowded nodes (used to place the single-visitor kernel on the roofline).
    "wide": dict(n_trees=32768, nodes_per_tree=1000, dense=1, fanout=225, legal_frac=0.5, last_legal=0, zipf_s=1.2,
                 n_cap=10_000, logit_sigma=1.0, max_depth=12, growth_width=8, n_traversals=32768, c_puct=1.4,
                 virtual_loss=3),
}


def _lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "libomk_synth.so")
        if not os.path.exists(so):
            raise OSError("%s is missing: build it with `python -m omoknuni_small_amd.build`" % so)
        _LIB = C.CDLL(so)
        _LIB.omk_synth_generate.restype = C.c_int
    return _LIB


def generate(config, seed=2025, nodes_per_tree=None, n_trees=None, **overrides):
    """Returns (soa, roots, meta).  `config` is a name from CONFIGS or a dict of the same keys;
    nodes_per_tree / n_trees / any other key override it (used to scale a workload down)."""
    cfg = dict(CONFIGS[config]) if isinstance(config, str) else dict(config)
    if nodes_per_tree is not None:
        cfg["nodes_per_tree"] = int(nodes_per_tree)
    if n_trees is not None:
        cfg["n_trees"] = int(n_trees)
    cfg.update(overrides)
    nt, npt = cfg["n_trees"], cfg["nodes_per_tree"]
    total = nt * npt
    dense = int(cfg.get("dense", 1))
    rave = int(cfg.get("has_rave", 0))
    with_hash = int(cfg.get("with_hash", 0))
    soa = dict(N=np.empty(total, np.int32), W=np.empty(total, np.float32), P=np.empty(total, np.float32),
               VL=np.empty(total, np.int32), child_begin=np.empty(total, np.int32),
               child_count=np.empty(total, np.int32), action=np.empty(total, np.int32))
    if rave:
        soa["rN"] = np.empty(total, np.int32)
        soa["rW"] = np.empty(total, np.float32)
    if dense:
        soa["legal"] = np.zeros((total + 31) // 32, np.uint32)
    if with_hash:
        soa["hash"] = np.empty(total, np.uint64)
    depth = np.empty(total, np.int32)
    roots = np.empty(nt, np.int32)
    used = np.empty(nt, np.int64)
    desc = _Desc(nt, npt, dense, int(cfg.get("fanout", 0)), float(cfg.get("legal_frac", 1.0)),
                 int(cfg.get("last_legal", 0)), float(cfg.get("poisson_lambda", 0.0)), int(cfg.get("fan_min", 1)),
                 int(cfg.get("fan_max", 1)), float(cfg["zipf_s"]), int(cfg["n_cap"]), float(cfg["logit_sigma"]),
                 int(cfg["max_depth"]), int(cfg["growth_width"]), rave, int(cfg.get("sort_by_prior", 0)),
                 int(cfg.get("pw", 0)), with_hash, float(cfg.get("c_puct", 1.4)), int(cfg.get("virtual_loss", 3)),
                 int(seed))

    def p(a):
        return a.ctypes.data if a is not None else None

    out = _Out(p(soa["N"]), p(soa["W"]), p(soa["P"]), p(soa["VL"]), p(soa.get("rN")), p(soa.get("rW")),
               p(soa["child_begin"]), p(soa["child_count"]), p(soa["action"]), p(soa.get("legal")),
               p(soa.get("hash")), p(depth), p(roots), p(used))
    rc = _lib().omk_synth_generate(C.byref(desc), C.byref(out))
    if rc != 0:
        raise ValueError("omk_synth_generate rejected the configuration")
    meta = dict(cfg)
    meta.update(seed=int(seed), n_nodes=total, used=used, depth=depth)
    return soa, roots, meta


def traversal_roots(roots, n_traversals):
    """Root of every traversal of a step: traversal t descends tree t % n_trees."""
    return np.ascontiguousarray(roots[np.arange(n_traversals) % len(roots)], dtype=np.int32)
