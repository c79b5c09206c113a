"""ctypes binding of the CPU checker (libref_cpu.so).

TEST INFRASTRUCTURE ONLY: imported by tests, by the smoke check and by the
benchmark's cpu_baseline leg, never by the shipped package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

i32p = C.POINTER(C.c_int32)
f32p = C.POINTER(C.c_float)
u32p = C.POINTER(C.c_uint32)
u64p = C.POINTER(C.c_uint64)


class _Tree(C.Structure):
    _fields_ = [("n_nodes", C.c_int64), ("N", i32p), ("W", f32p), ("P", f32p), ("VL", i32p),
                ("rN", i32p), ("rW", f32p), ("child_begin", i32p), ("child_count", i32p),
                ("action", i32p), ("legal", u32p)]


class _Params(C.Structure):
    _fields_ = [("c_puct", C.c_float), ("virtual_loss", C.c_int32), ("use_rave", C.c_int32),
                ("rave_k", C.c_float), ("pw", C.c_int32), ("max_depth", C.c_int32)]


class _Info(C.Structure):
    _fields_ = [("best", C.c_float), ("second", C.c_float), ("n_candidates", C.c_int32),
                ("near_tie", C.c_int32)]


TT_SLOT = np.dtype([("key", "<u8"), ("node", "<i4"), ("depth", "<i4")])


def build(force=False):
    so = os.path.join(_HERE, "libref_cpu.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libref_cpu.so"])
    return so


def lib():
    global _LIB
    if _LIB is None:
        L = C.CDLL(build())
        L.ref_widened_children.restype = C.c_int32
        L.ref_widened_children.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_float, C.c_float]
        L.ref_combined_value.restype = C.c_float
        L.ref_combined_value.argtypes = [C.POINTER(_Tree), C.c_int32, C.c_float]
        L.ref_child_scores.argtypes = [C.POINTER(_Tree), C.c_int32, C.c_int32, C.POINTER(_Params), f32p, f32p]
        L.ref_ceil_sqrt.restype = C.c_int32
        L.ref_ceil_sqrt.argtypes = [C.c_int32]
        L.ref_select_child.restype = C.c_int32
        L.ref_select_child.argtypes = [C.POINTER(_Tree), C.c_int32, C.POINTER(_Params), C.POINTER(_Info)]
        for name in ("ref_add_vl", "ref_remove_vl"):
            getattr(L, name).argtypes = [C.POINTER(_Tree), C.c_int32, C.c_int32]
            getattr(L, name).restype = None
        L.ref_remove_vl1.argtypes = [C.POINTER(_Tree), C.c_int32]
        L.ref_remove_vl1.restype = None
        L.ref_update.argtypes = [C.POINTER(_Tree), C.c_int32, C.c_float]
        L.ref_update.restype = None
        L.ref_select_batch.restype = C.c_int
        L.ref_select_batch.argtypes = [C.POINTER(_Tree), i32p, C.c_int32, C.POINTER(_Params), i32p, i32p, i32p, i32p]
        for name in ("ref_apply_vl_paths", "ref_revert_vl_paths"):
            getattr(L, name).argtypes = [C.POINTER(_Tree), i32p, i32p, C.c_int32, C.c_int32, C.c_int32]
            getattr(L, name).restype = None
        L.ref_backup_batch.argtypes = [C.POINTER(_Tree), i32p, i32p, f32p, C.c_int32, C.c_int32, C.c_int32]
        L.ref_backup_batch.restype = None
        L.ref_gather_actions.argtypes = [C.POINTER(_Tree), i32p, i32p, C.c_int32, C.c_int32, i32p]
        L.ref_gather_actions.restype = None
        L.ref_tt_clear.argtypes = [C.c_void_p, C.c_int32]
        L.ref_tt_clear.restype = None
        L.ref_tt_insert.argtypes = [C.c_void_p, C.c_int32, C.c_uint64, C.c_int32, C.c_int32]
        L.ref_tt_insert.restype = C.c_int
        L.ref_tt_probe.argtypes = [C.c_void_p, C.c_int32, u64p, C.c_int64, C.c_int32, i32p]
        L.ref_tt_probe.restype = C.c_int64
        L.ref_zobrist_tables.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_uint32, u64p, u64p]
        L.ref_zobrist_tables.restype = C.c_int
        L.ref_position_key.argtypes = [C.c_void_p, C.c_int32, u64p, C.c_int64, u64p, C.c_int32]
        L.ref_position_key.restype = C.c_uint64
        L.ref_leaf_keys.argtypes = [C.POINTER(_Tree), i32p, i32p, C.c_int32, C.c_int32, C.c_void_p, i32p, C.c_int32,
                                    u64p, C.c_int64, u64p, u64p]
        L.ref_leaf_keys.restype = C.c_int32
        L.ref_mt64_seed.argtypes = [C.c_void_p, C.c_uint64]
        L.ref_mt64_seed.restype = None
        L.ref_mt64_next.argtypes = [C.c_void_p]
        L.ref_mt64_next.restype = C.c_uint64
        _LIB = L
    return _LIB


def _ptr(a, ty):
    return a.ctypes.data_as(ty) if a is not None else ty()


def make_params(c_puct=1.4, virtual_loss=3, use_rave=False, rave_k=3000.0, pw=False, max_depth=32):
    return _Params(c_puct, int(virtual_loss), int(bool(use_rave)), rave_k, int(bool(pw)), int(max_depth))


class RefTree:
    """Owns private copies of the per-node arrays and runs the checker on them."""

    def __init__(self, N, W, P, VL, child_begin, child_count, action=None, rN=None, rW=None, legal=None):
        n = len(N)
        self.n = n
        self.N = np.ascontiguousarray(N, dtype=np.int32).copy()
        self.W = np.ascontiguousarray(W, dtype=np.float32).copy()
        self.P = np.ascontiguousarray(P, dtype=np.float32).copy()
        self.VL = np.ascontiguousarray(VL, dtype=np.int32).copy()
        self.child_begin = np.ascontiguousarray(child_begin, dtype=np.int32).copy()
        self.child_count = np.ascontiguousarray(child_count, dtype=np.int32).copy()
        self.action = None if action is None else np.ascontiguousarray(action, dtype=np.int32).copy()
        self.rN = None if rN is None else np.ascontiguousarray(rN, dtype=np.int32).copy()
        self.rW = None if rW is None else np.ascontiguousarray(rW, dtype=np.float32).copy()
        self.legal = None if legal is None else np.ascontiguousarray(legal, dtype=np.uint32).copy()
        for a in (self.W, self.P, self.VL, self.child_begin, self.child_count):
            assert len(a) == n
        if self.legal is not None:
            assert len(self.legal) * 32 >= n
        self._c = _Tree(n, _ptr(self.N, i32p), _ptr(self.W, f32p), _ptr(self.P, f32p), _ptr(self.VL, i32p),
                        _ptr(self.rN, i32p), _ptr(self.rW, f32p), _ptr(self.child_begin, i32p),
                        _ptr(self.child_count, i32p), _ptr(self.action, i32p), _ptr(self.legal, u32p))

    @classmethod
    def from_soa(cls, soa):
        """soa: mapping with the keys of omoknuni_small_amd.synth (N, W, P, VL, child_begin, ...)."""
        return cls(soa["N"], soa["W"], soa["P"], soa["VL"], soa["child_begin"], soa["child_count"],
                   action=soa.get("action"), rN=soa.get("rN"), rW=soa.get("rW"), legal=soa.get("legal"))

    # -- single-node operations -------------------------------------------------
    def select_child(self, node, params, with_info=False):
        info = _Info()
        r = lib().ref_select_child(C.byref(self._c), int(node), C.byref(params), C.byref(info))
        if with_info:
            return r, dict(best=info.best, second=info.second, n_candidates=info.n_candidates,
                           near_tie=bool(info.near_tie))
        return r

    def child_scores(self, parent, child, params):
        a, b = C.c_float(), C.c_float()
        lib().ref_child_scores(C.byref(self._c), int(parent), int(child), C.byref(params), C.byref(a), C.byref(b))
        return np.float32(a.value), np.float32(b.value)

    def combined_value(self, node, rave_k):
        return np.float32(lib().ref_combined_value(C.byref(self._c), int(node), rave_k))

    def add_vl(self, node, amount):
        lib().ref_add_vl(C.byref(self._c), int(node), int(amount))

    def remove_vl(self, node, amount=None):
        if amount is None:
            lib().ref_remove_vl1(C.byref(self._c), int(node))
        else:
            lib().ref_remove_vl(C.byref(self._c), int(node), int(amount))

    def update(self, node, value):
        lib().ref_update(C.byref(self._c), int(node), float(value))

    # -- batched operations -----------------------------------------------------
    def select_batch(self, roots, params, near_ties=True):
        roots = np.ascontiguousarray(roots, dtype=np.int32)
        B = len(roots)
        stride = params.max_depth + 1
        paths = np.empty((B, stride), dtype=np.int32)
        path_len = np.empty(B, dtype=np.int32)
        leaf = np.empty(B, dtype=np.int32)
        nt = np.empty(B, dtype=np.int32) if near_ties else None
        rc = lib().ref_select_batch(C.byref(self._c), _ptr(roots, i32p), B, C.byref(params), _ptr(paths, i32p),
                                    _ptr(path_len, i32p), _ptr(leaf, i32p), _ptr(nt, i32p))
        if rc != 0:
            raise ValueError("ref_select_batch: bad root")
        return paths, path_len, leaf, nt

    def _paths_args(self, paths, path_len):
        paths = np.ascontiguousarray(paths, dtype=np.int32)
        path_len = np.ascontiguousarray(path_len, dtype=np.int32)
        return paths, path_len, paths.shape[0], paths.shape[1]

    def apply_vl_paths(self, paths, path_len, amount):
        paths, path_len, B, stride = self._paths_args(paths, path_len)
        lib().ref_apply_vl_paths(C.byref(self._c), _ptr(paths, i32p), _ptr(path_len, i32p), B, stride, int(amount))

    def revert_vl_paths(self, paths, path_len, amount):
        paths, path_len, B, stride = self._paths_args(paths, path_len)
        lib().ref_revert_vl_paths(C.byref(self._c), _ptr(paths, i32p), _ptr(path_len, i32p), B, stride, int(amount))

    def backup_batch(self, paths, path_len, values, amount):
        paths, path_len, B, stride = self._paths_args(paths, path_len)
        values = np.ascontiguousarray(values, dtype=np.float32)
        assert len(values) == B
        lib().ref_backup_batch(C.byref(self._c), _ptr(paths, i32p), _ptr(path_len, i32p), _ptr(values, f32p),
                               B, stride, int(amount))

    def expand_batch(self, leaf, move_begin, moves, policy=None, action_space=0, policy_begin=None, widening=None):
        """MCTSNode::expand + setPriorProbabilities for the leaves of a batch (see ref_cpu.h).
        Grows the arrays; returns first_child per traversal (-1 where nothing was added).
        policy_begin: ragged policies (policy is then their concatenation); widening: (c, k) of
        progressive widening, None = off."""
        leaf = np.ascontiguousarray(leaf, dtype=np.int32)
        move_begin = np.ascontiguousarray(move_begin, dtype=np.int32)
        moves = np.ascontiguousarray(moves, dtype=np.int32)
        B = len(leaf)
        cap = self.n + int(np.minimum(np.diff(move_begin), 1000).clip(min=0).sum())

        def grow(a, dtype, n=cap):
            if a is None:
                return None
            out = np.zeros(n, dtype=dtype)
            out[:len(a)] = a
            return out

        self.N, self.W, self.P, self.VL = (grow(self.N, np.int32), grow(self.W, np.float32),
                                           grow(self.P, np.float32), grow(self.VL, np.int32))
        self.rN, self.rW = grow(self.rN, np.int32), grow(self.rW, np.float32)
        self.child_begin, self.child_count = grow(self.child_begin, np.int32), grow(self.child_count, np.int32)
        self.action = grow(self.action, np.int32)
        self.legal = grow(self.legal, np.uint32, (cap + 31) // 32)
        if self.legal is not None and self.n & 31:
            self.legal[self.n >> 5] &= np.uint32((1 << (self.n & 31)) - 1)  # bits of ids that do not exist yet
        pol = None if policy is None else np.ascontiguousarray(policy, dtype=np.float32).reshape(-1)
        if pol is not None and len(pol) == 0:
            pol = np.zeros(1, np.float32)
        pb = None
        if pol is not None:
            pb = (np.arange(B + 1, dtype=np.int32) * int(action_space) if policy_begin is None
                  else np.ascontiguousarray(policy_begin, dtype=np.int32))
        first = np.empty(B, dtype=np.int32)
        fn = lib().ref_expand_batch_ex
        fn.restype = C.c_int64
        use_pw, cpw, kpw = (0, 0.0, 0.0) if widening is None else (1, float(widening[0]), float(widening[1]))
        n_after = fn(C.c_int64(self.n), C.c_int64(cap), _ptr(self.N, i32p), _ptr(self.W, f32p), _ptr(self.P, f32p),
                     _ptr(self.VL, i32p), _ptr(self.rN, i32p), _ptr(self.rW, f32p), _ptr(self.child_begin, i32p),
                     _ptr(self.child_count, i32p), _ptr(self.action, i32p), _ptr(self.legal, u32p), _ptr(leaf, i32p),
                     B, _ptr(move_begin, i32p), _ptr(moves, i32p), _ptr(pb, i32p), _ptr(pol, f32p), int(action_space),
                     C.c_int32(use_pw), C.c_float(cpw), C.c_float(kpw), _ptr(first, i32p))
        assert n_after >= 0
        self.n = int(n_after)
        for name in ("N", "W", "P", "VL", "rN", "rW", "child_begin", "child_count", "action"):
            a = getattr(self, name)
            if a is not None:
                setattr(self, name, a[:self.n].copy())
        if self.legal is not None:
            self.legal = self.legal[:(self.n + 31) // 32].copy()
        self._c = _Tree(self.n, _ptr(self.N, i32p), _ptr(self.W, f32p), _ptr(self.P, f32p), _ptr(self.VL, i32p),
                        _ptr(self.rN, i32p), _ptr(self.rW, f32p), _ptr(self.child_begin, i32p),
                        _ptr(self.child_count, i32p), _ptr(self.action, i32p), _ptr(self.legal, u32p))
        return first

    def rave_backup_batch(self, paths, path_len, values):
        paths, path_len, B, stride = self._paths_args(paths, path_len)
        values = np.ascontiguousarray(values, dtype=np.float32)
        lib().ref_rave_backup_batch(C.byref(self._c), _ptr(paths, i32p), _ptr(path_len, i32p), _ptr(values, f32p),
                                    B, stride)

    def reroot_child(self, root, last_action):
        return int(lib().ref_reroot_child(C.byref(self._c), int(root), int(last_action)))

    def compacted(self, new_root):
        """The subtree of new_root as a new RefTree with ids 0..k-1 (breadth-first, sibling order
        kept) and the old id of every new node."""
        order = np.empty(self.n, dtype=np.int32)
        fn = lib().ref_compact_order
        fn.restype = C.c_int64
        k = int(fn(C.byref(self._c), int(new_root), _ptr(order, i32p)))
        order = order[:k].copy()
        # first child of new node i: children were appended in visiting order
        cc = self.child_count[order]
        cb = np.zeros(k, np.int32)
        cb[cc > 0] = (1 + np.concatenate([[0], np.cumsum(cc)[:-1]]))[cc > 0]
        legal = None
        if self.legal is not None:
            bits = (self.legal[order >> 5] >> (order & 31).astype(np.uint32)) & 1
            pad = np.zeros((k + 31) // 32 * 32, np.uint8)
            pad[:k] = bits
            legal = np.packbits(pad.reshape(-1, 32), axis=1, bitorder="little").view("<u4").reshape(-1).copy()
        t = RefTree(self.N[order], self.W[order], self.P[order], self.VL[order], cb, cc,
                    action=None if self.action is None else self.action[order],
                    rN=None if self.rN is None else self.rN[order], rW=None if self.rW is None else self.rW[order],
                    legal=legal)
        return t, order

    def action_probabilities(self, root, temperature, action_space):
        """MCTSEngine::getActionProbabilities over the root's children; (probabilities, children)."""
        out = np.empty(int(action_space), dtype=np.float32)
        n = lib().ref_action_probabilities(C.byref(self._c), int(root), C.c_float(temperature), int(action_space),
                                           _ptr(out, f32p))
        return out, int(n)

    def add_root_noise(self, root, gamma, epsilon):
        """MCTSEngine::addDirichletNoise from the gamma samples on; returns the number of children."""
        gamma = np.ascontiguousarray(gamma, dtype=np.float32)
        L = lib()
        L.ref_add_root_noise.restype = C.c_int32
        n = L.ref_add_root_noise(C.byref(self._c), C.c_int32(int(root)), _ptr(gamma, f32p), C.c_int32(len(gamma)),
                                 C.c_float(epsilon))
        assert n >= 0, "sample count does not match the number of children"
        return int(n)

    def select_redirect_batch(self, roots, params, tt, node_key, alias=None):
        """The traversal loop with the transposition table on, redirects included (see ref_cpu.c).
        alias (int32 per node, -1 = the slot holds its own node) is updated in place; returns
        (paths, path_len, leaf, moves, counts) with counts = new entries, replacements, lookups that found
        an entry, redirects, steps; tt's clock advances as the reference's access counter does on one thread."""
        roots = np.ascontiguousarray(roots, dtype=np.int32)
        node_key = np.ascontiguousarray(node_key, dtype=np.uint64)
        assert len(node_key) == self.n
        if alias is None:
            alias = np.full(self.n, -1, np.int32)
        assert alias.dtype == np.int32 and len(alias) == self.n and alias.flags.c_contiguous
        B = len(roots)
        stride = params.max_depth + 1
        paths = np.empty((B, stride), dtype=np.int32)
        path_len = np.empty(B, dtype=np.int32)
        leaf = np.empty(B, dtype=np.int32)
        moves = np.empty((B, params.max_depth), dtype=np.int32)
        counts = np.zeros(6, np.int32)
        fn = lib().ref_select_redirect_batch
        fn.restype = C.c_int
        rc = fn(C.byref(self._c), _ptr(alias, i32p), _ptr(roots, i32p), C.c_int32(B), C.byref(params),
                C.c_void_p(tt.slots.ctypes.data), C.c_void_p(tt.meta.ctypes.data), C.c_int32(tt.log2),
                C.c_uint32(tt.clock & 0xFFFFFFFF), C.c_float(tt.threshold), _ptr(node_key, u64p), _ptr(paths, i32p),
                _ptr(path_len, i32p), _ptr(leaf, i32p), _ptr(moves, i32p), _ptr(counts, i32p))
        if rc == -2:
            # the table ran full: every traversal was still made (without the entries that found no room);
            # the error carries what they did
            tt.clock += int(counts[5])
            err = ValueError("ref_select_redirect_batch: table full")
            err.result = (paths, path_len, leaf, moves, counts[:5])
            raise err
        if rc != 0:
            raise ValueError("ref_select_redirect_batch: %d" % rc)
        tt.clock += int(counts[5])
        return paths, path_len, leaf, moves, counts[:5]

    def gather_actions(self, paths, path_len):
        paths, path_len, B, stride = self._paths_args(paths, path_len)
        out = np.empty((B, stride - 1), dtype=np.int32)
        lib().ref_gather_actions(C.byref(self._c), _ptr(paths, i32p), _ptr(path_len, i32p), B, stride, _ptr(out, i32p))
        return out


TT_META = np.dtype([("visits", "<u4"), ("value", "<f4"), ("last_access", "<u4"), ("reserved", "<i4")])


class RefTT:
    def __init__(self, log2_slots):
        self.log2 = int(log2_slots)
        self.slots = np.empty(1 << self.log2, dtype=TT_SLOT)
        self.meta = np.zeros(1 << self.log2, dtype=TT_META)
        self.clock = 0          # entry i of a call has the time clock + i; every call advances it by its length
        self.threshold = 0.1    # Config::replacement_threshold
        lib().ref_tt_clear(self.slots.ctypes.data, self.log2)

    def store(self, tree, keys, nodes, depths=None):
        """store() with the replacement policy for a batch; (new entries, replacements, duplicates dropped)."""
        keys = np.ascontiguousarray(keys, np.uint64)
        nodes = np.ascontiguousarray(nodes, np.int32)
        dp = None if depths is None else np.ascontiguousarray(depths, np.int32)
        counts = np.zeros(4, np.int32)
        fn = lib().ref_tt_store_batch
        fn.restype = C.c_int
        rc = fn(C.c_void_p(self.slots.ctypes.data), C.c_void_p(self.meta.ctypes.data), C.c_int32(self.log2),
                C.byref(tree._c), _ptr(keys, u64p), _ptr(nodes, i32p), _ptr(dp, i32p), C.c_int64(len(keys)),
                C.c_uint32(self.clock & 0xFFFFFFFF), C.c_float(self.threshold), _ptr(counts, i32p))
        self.clock += len(keys)
        assert rc == 0, rc
        return tuple(int(x) for x in counts[:3])

    def lookup(self, keys, min_depth=0):
        """lookup() for a batch, stamping the entries it finds; (nodes, hits)."""
        keys = np.ascontiguousarray(keys, np.uint64)
        out = np.empty(len(keys), np.int32)
        fn = lib().ref_tt_lookup_batch
        fn.restype = C.c_int64
        hits = fn(C.c_void_p(self.slots.ctypes.data), C.c_void_p(self.meta.ctypes.data), C.c_int32(self.log2),
                  _ptr(keys, u64p), C.c_int64(len(keys)), C.c_int32(int(min_depth)), C.c_uint32(self.clock & 0xFFFFFFFF),
                  _ptr(out, i32p))
        self.clock += len(keys)
        return out, int(hits)

    def traverse(self, tree, paths, path_len, step_keys):
        """The table's part of the traversal loop (mcts_engine_batch_tree_simple.cpp:116-162) over row-major
        paths: step_keys [B, D] = key of the state after step d + 1 of traversal t.  Stores the selected
        children without visits, looks every step up; returns (hits [B, D] node or -1, counts)."""
        B, row = paths.shape
        D = row - 1
        d_idx = np.arange(1, row)[None, :]
        valid = d_idx < path_len[:, None]
        step_nodes = np.where(valid, paths[:, 1:], -1).astype(np.int32)
        keys = np.where(valid, step_keys, np.uint64(0xFFFFFFFFFFFFFFFF)).astype(np.uint64)
        unvisited = valid & (tree.N[np.maximum(step_nodes, 0)] == 0)
        store_nodes = np.where(unvisited, step_nodes, -1).astype(np.int32)
        depths = np.broadcast_to(d_idx, (B, D)).astype(np.int32)
        new, repl, dup = self.store(tree, keys.reshape(-1), store_nodes.reshape(-1), depths.reshape(-1))
        found, _ = self.lookup(keys.reshape(-1))
        found = found.reshape(B, D)
        hit = valid & (found >= 0) & (found != step_nodes) & (tree.N[np.maximum(found, 0)] > 0)
        hits = np.where(hit, found, -1).astype(np.int32)
        return hits, (new, repl, dup, int(hit.sum()))

    def insert(self, key, node, depth=0):
        return lib().ref_tt_insert(self.slots.ctypes.data, self.log2, int(key), int(node), int(depth))

    def probe(self, keys, min_depth=0):
        keys = np.ascontiguousarray(keys, dtype=np.uint64)
        out = np.empty(len(keys), dtype=np.int32)
        hits = lib().ref_tt_probe(self.slots.ctypes.data, self.log2, _ptr(keys, u64p), len(keys), int(min_depth),
                                  _ptr(out, i32p))
        return out, int(hits)


def mt19937_64(seed, count):
    """The first `count` outputs of std::mt19937_64(seed)."""
    g = (C.c_uint64 * 313)()
    lib().ref_mt64_seed(g, int(seed))
    return np.array([lib().ref_mt64_next(g) for _ in range(count)], dtype=np.uint64)


def zobrist_tables(board_size, n_piece, n_players, seed):
    """piece [n_piece, board_size**2], player [n_players] of ZobristHash(board_size, n_piece, n_players, seed)."""
    piece = np.empty((n_piece, board_size * board_size), np.uint64)
    player = np.empty(n_players, np.uint64)
    rc = lib().ref_zobrist_tables(int(board_size), int(n_piece), int(n_players), int(seed), _ptr(piece, u64p),
                                  _ptr(player, u64p))
    if rc != 0:
        raise ValueError("arguments the ZobristHash constructor rejects, or seed 0")
    return piece, player


def position_key(board, piece, player, current_player):
    """compute_hash_signature_internal of a board (0 empty, 1 BLACK, 2 WHITE) with `current_player` to move."""
    board = np.ascontiguousarray(board, np.int8)
    piece = np.ascontiguousarray(piece, np.uint64)
    player = np.ascontiguousarray(player, np.uint64)
    return int(lib().ref_position_key(board.ctypes.data, len(board), _ptr(piece, u64p), piece.shape[1],
                                      _ptr(player, u64p), int(current_player)))


def leaf_keys(tree, paths, path_len, root_boards, root_player, piece, player):
    """getHash() of every path's replayed state; (keys, number of bad paths)."""
    paths = np.ascontiguousarray(paths, np.int32)
    path_len = np.ascontiguousarray(path_len, np.int32)
    root_boards = np.ascontiguousarray(root_boards, np.int8)
    root_player = np.ascontiguousarray(root_player, np.int32)
    piece = np.ascontiguousarray(piece, np.uint64)
    player = np.ascontiguousarray(player, np.uint64)
    B, cells = root_boards.shape
    out = np.empty(B, np.uint64)
    bad = lib().ref_leaf_keys(C.byref(tree._c), _ptr(paths, i32p), _ptr(path_len, i32p), B, paths.shape[1],
                              root_boards.ctypes.data, _ptr(root_player, i32p), cells, _ptr(piece, u64p),
                              piece.shape[1], _ptr(player, u64p), _ptr(out, u64p))
    return out, int(bad)
