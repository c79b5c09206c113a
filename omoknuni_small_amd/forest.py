"""Host-side mirror of the C ABI in include/omk_forest.h.

The classes follow the phases of the reference's MCTSEngine::executeBatchedTreeSearch
(src/mcts/mcts_engine_batch_tree_simple.cpp): Batch.select() is phase 1 (selectChild +
applyVirtualLoss down to a leaf), Batch.read() is the leaf gather, Batch.backup() is
phase 3 (update + revertVirtualLoss, sign flipped per ply).  Every call goes through
libomk_forest.so; there is no host fallback, and loading fails loudly when the library
has not been built.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

i32p = C.POINTER(C.c_int32)
f32p = C.POINTER(C.c_float)
u32p = C.POINTER(C.c_uint32)
u64p = C.POINTER(C.c_uint64)

EXPORTS = [
    "omk_last_error", "omk_version", "omk_forest_create", "omk_forest_destroy", "omk_forest_set_stream", "omk_forest_get_stream",
    "omk_forest_upload", "omk_forest_download", "omk_forest_node_count", "omk_forest_download_structure",
    "omk_expand_batch", "omk_expand_batch_ex", "omk_forest_action_probabilities", "omk_forest_add_root_noise", "omk_forest_set_keys", "omk_forest_reroot_child", "omk_forest_compact", "omk_forest_compact_static",
    "omk_sync", "omk_batch_create", "omk_batch_destroy",
    "omk_batch_set_roots", "omk_batch_set_values", "omk_batch_device", "omk_select_batch", "omk_backup_batch",
    "omk_revert_vl", "omk_backup_rave_batch", "omk_apply_vl_paths", "omk_revert_vl_paths", "omk_backup_paths", "omk_batch_read",
    "omk_batch_leaf_keys", "omk_debug_trace", "omk_batch_set_trace", "omk_batch_truncated", "omk_batch_stats", "omk_batch_set_stats", "omk_batch_set_spin_limit", "omk_debug_set_select_count", "omk_tt_create", "omk_tt_destroy", "omk_tt_clear", "omk_tt_insert", "omk_tt_probe",
    "omk_tt_probe_leaves", "omk_tt_store", "omk_tt_set_replacement_threshold", "omk_tt_traverse", "omk_tt_select_redirect", "omk_forest_download_redirects", "omk_tt_download_meta", "omk_tt_upload", "omk_tt_download", "omk_dev_alloc", "omk_dev_free", "omk_dev_h2d",
    "omk_dev_d2h", "omk_dev_copy", "omk_soa_count_legal", "omk_soa_compact_legal",
]

TT_SLOT = np.dtype([("key", "<u8"), ("node", "<i4"), ("depth", "<i4")])
TT_META = np.dtype([("visits", "<u4"), ("value", "<f4"), ("last_access", "<u4"), ("reserved", "<i4")])


class OmkError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("omk status %d: %s" % (code, message))
        self.code = code


class _SoaView(C.Structure):
    _fields_ = [("n_nodes", C.c_int64), ("N", i32p), ("W", f32p), ("P", f32p), ("VL", i32p), ("rN", i32p),
                ("rW", f32p), ("child_begin", i32p), ("child_count", i32p), ("action", i32p), ("legal", u32p),
                ("hash", u64p)]


class _ForestDesc(C.Structure):
    _fields_ = [("capacity_nodes", C.c_int64), ("device", C.c_int32), ("has_rave", C.c_int32)]


class SelectParams(C.Structure):
    """MCTSSettings fields read on this path (reference include/mcts/mcts_engine.h:81-112)."""
    _fields_ = [("c_puct", C.c_float), ("virtual_loss", C.c_int32), ("use_rave", C.c_int32),
                ("rave_k", C.c_float), ("pw", C.c_int32)]

    def __init__(self, c_puct=1.4, virtual_loss=3, use_rave=False, rave_k=3000.0, pw=False):
        super().__init__(c_puct, int(virtual_loss), int(bool(use_rave)), rave_k, int(bool(pw)))


class _ExpandParams(C.Structure):
    """MCTSSettings fields MCTSNode::expand reads (reference include/mcts/mcts_engine.h:98-103)."""
    _fields_ = [("action_space", C.c_int32), ("use_progressive_widening", C.c_int32),
                ("progressive_widening_c", C.c_float), ("progressive_widening_k", C.c_float)]


class _BatchDev(C.Structure):
    _fields_ = [("d_paths", C.c_void_p), ("d_path_len", C.c_void_p), ("d_leaf", C.c_void_p),
                ("d_values", C.c_void_p), ("stride", C.c_int32), ("max_depth", C.c_int32),
                ("n_traversals", C.c_int32)]


def library_path():
    """libomk_forest.so beside this file, or another build of the same ABI named by OMK_FOREST_LIB."""
    return os.environ.get("OMK_FOREST_LIB") or os.path.join(_HERE, "libomk_forest.so")


def load_library():
    """Loads libomk_forest.so; raises when it is missing rather than falling back to anything."""
    global _LIB
    if _LIB is not None:
        return _LIB
    so = library_path()
    if not os.path.exists(so):
        raise OSError("%s is missing: build it with `python -m omoknuni_small_amd.build` "
                      "(there is no host fallback for the HIP path)" % so)
    L = C.CDLL(so)
    L.omk_last_error.restype = C.c_char_p
    for name in EXPORTS:
        if name != "omk_last_error":
            getattr(L, name).restype = C.c_int
    L.omk_soa_count_legal.restype = C.c_int64
    _LIB = L
    return L


def _check(rc):
    if rc != 0:
        raise OmkError(rc, load_library().omk_last_error().decode())


def _ptr(a, ty):
    return a.ctypes.data_as(ty) if a is not None else ty()


def _arr(x, dtype):
    return None if x is None else np.ascontiguousarray(x, dtype=dtype)


def _view_of(keep):
    return _SoaView(len(keep["N"]), _ptr(keep["N"], i32p), _ptr(keep["W"], f32p), _ptr(keep["P"], f32p),
                    _ptr(keep["VL"], i32p), _ptr(keep["rN"], i32p), _ptr(keep["rW"], f32p),
                    _ptr(keep["child_begin"], i32p), _ptr(keep["child_count"], i32p), _ptr(keep["action"], i32p),
                    _ptr(keep["legal"], u32p), _ptr(keep["hash"], u64p))


def compact_legal(soa):
    """A forest with one slot per action and a legal mask, re-laid without its empty slots
    (omk_soa_compact_legal; host only).  Returns (soa without a mask, old_to_new, new_to_old)."""
    lib = load_library()
    keep = dict(N=_arr(soa["N"], np.int32), W=_arr(soa["W"], np.float32), P=_arr(soa["P"], np.float32),
                VL=_arr(soa["VL"], np.int32), rN=_arr(soa.get("rN"), np.int32), rW=_arr(soa.get("rW"), np.float32),
                child_begin=_arr(soa["child_begin"], np.int32), child_count=_arr(soa["child_count"], np.int32),
                action=_arr(soa.get("action"), np.int32), legal=_arr(soa.get("legal"), np.uint32),
                hash=_arr(soa.get("hash"), np.uint64))
    n = len(keep["N"])
    if keep["legal"] is not None and len(keep["legal"]) * 32 < n:
        raise ValueError("legal mask shorter than the node count")
    v = _view_of(keep)
    cnt = int(lib.omk_soa_count_legal(C.byref(v)))
    if cnt < 0:
        _check(cnt)
    out = dict(N=np.empty(cnt, np.int32), W=np.empty(cnt, np.float32), P=np.empty(cnt, np.float32),
               VL=np.empty(cnt, np.int32), child_begin=np.empty(cnt, np.int32), child_count=np.empty(cnt, np.int32),
               action=np.empty(cnt, np.int32))
    for k, dt in (("rN", np.int32), ("rW", np.float32), ("hash", np.uint64)):
        out[k] = np.empty(cnt, dt) if keep[k] is not None else None
    old_to_new, new_to_old = np.empty(n, np.int32), np.empty(cnt, np.int32)
    _check(lib.omk_soa_compact_legal(C.byref(v), C.c_int64(cnt), _ptr(out["N"], i32p), _ptr(out["W"], f32p),
                                     _ptr(out["P"], f32p), _ptr(out["VL"], i32p), _ptr(out["rN"], i32p),
                                     _ptr(out["rW"], f32p), _ptr(out["child_begin"], i32p),
                                     _ptr(out["child_count"], i32p), _ptr(out["action"], i32p),
                                     _ptr(out["hash"], u64p), _ptr(old_to_new, i32p), _ptr(new_to_old, i32p)))
    return {k: a for k, a in out.items() if a is not None}, old_to_new, new_to_old


class Forest:
    """Device-resident forest: the per-node arrays that replace the MCTSNode pointer tree."""

    def __init__(self, capacity_nodes, device=0, has_rave=False):
        self._lib = load_library()
        self._h = C.c_void_p()
        self.has_rave = bool(has_rave)
        self.n_nodes = 0
        desc = _ForestDesc(int(capacity_nodes), int(device), int(self.has_rave))
        _check(self._lib.omk_forest_create(C.byref(desc), C.byref(self._h)))

    @classmethod
    def from_soa(cls, soa, device=0, capacity=None):
        """capacity > len(N) leaves room for Batch.expand() to add nodes."""
        f = cls(max(len(soa["N"]), int(capacity or 0)), device=device, has_rave=soa.get("rN") is not None)
        f.upload(soa)
        return f

    def close(self):
        if self._h:
            self._lib.omk_forest_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_stream(self, hip_stream):
        _check(self._lib.omk_forest_set_stream(self._h, C.c_void_p(hip_stream or 0)))

    def get_stream(self):
        s = C.c_void_p()
        _check(self._lib.omk_forest_get_stream(self._h, C.byref(s)))
        return s.value or 0

    def sync(self):
        _check(self._lib.omk_sync(self._h))

    def upload(self, soa):
        keep = dict(N=_arr(soa["N"], np.int32), W=_arr(soa["W"], np.float32), P=_arr(soa["P"], np.float32),
                    VL=_arr(soa["VL"], np.int32), rN=_arr(soa.get("rN"), np.int32), rW=_arr(soa.get("rW"), np.float32),
                    child_begin=_arr(soa["child_begin"], np.int32), child_count=_arr(soa["child_count"], np.int32),
                    action=_arr(soa.get("action"), np.int32), legal=_arr(soa.get("legal"), np.uint32),
                    hash=_arr(soa.get("hash"), np.uint64))
        n = len(keep["N"])
        for k in ("W", "P", "VL", "child_begin", "child_count", "rN", "rW", "action", "hash"):
            if keep[k] is not None and len(keep[k]) != n:
                raise ValueError("array %s has %d entries, N has %d" % (k, len(keep[k]), n))
        if keep["legal"] is not None and len(keep["legal"]) * 32 < n:
            raise ValueError("legal mask shorter than the node count")
        v = _SoaView(n, _ptr(keep["N"], i32p), _ptr(keep["W"], f32p), _ptr(keep["P"], f32p), _ptr(keep["VL"], i32p),
                     _ptr(keep["rN"], i32p), _ptr(keep["rW"], f32p), _ptr(keep["child_begin"], i32p),
                     _ptr(keep["child_count"], i32p), _ptr(keep["action"], i32p), _ptr(keep["legal"], u32p),
                     _ptr(keep["hash"], u64p))
        _check(self._lib.omk_forest_upload(self._h, C.byref(v)))
        self.n_nodes = n

    def node_count(self):
        """(nodes now, capacity): the forest grows with Batch.expand()."""
        n, cap = C.c_int64(), C.c_int64()
        _check(self._lib.omk_forest_node_count(self._h, C.byref(n), C.byref(cap)))
        self.n_nodes = int(n.value)
        return int(n.value), int(cap.value)

    def reroot_child(self, root, last_action):
        """searchWithTreeReuse: the first child of root reached by last_action, or -1."""
        c = C.c_int32()
        _check(self._lib.omk_forest_reroot_child(self._h, C.c_int32(int(root)), C.c_int32(int(last_action)),
                                                 C.byref(c)))
        return int(c.value)

    def compact(self, new_root, static=False):
        """Keeps the subtree of new_root, renumbered breadth-first from 0; returns the old id of
        every new node.  static: the variant that allocates nothing (at most 2^20 nodes)."""
        n_old, _ = self.node_count()
        order = np.empty(n_old, np.int32)
        k = C.c_int64()
        fn = self._lib.omk_forest_compact_static if static else self._lib.omk_forest_compact
        _check(fn(self._h, C.c_int32(int(new_root)), C.byref(k), _ptr(order, i32p)))
        self.n_nodes = int(k.value)
        return order[:self.n_nodes].copy()

    def action_probabilities(self, root, temperature, action_space):
        """MCTSEngine::getActionProbabilities from the root's children; (probabilities, children)."""
        out = np.empty(int(action_space), np.float32)
        n = C.c_int32()
        _check(self._lib.omk_forest_action_probabilities(self._h, C.c_int32(int(root)), C.c_float(temperature),
                                                         C.c_int32(int(action_space)), _ptr(out, f32p), C.byref(n)))
        return out, int(n.value)

    def add_root_noise(self, root, gamma, epsilon):
        """MCTSEngine::addDirichletNoise: one caller-drawn gamma(alpha, 1) sample per child of `root`."""
        gamma = np.ascontiguousarray(gamma, dtype=np.float32)
        _check(self._lib.omk_forest_add_root_noise(self._h, C.c_int32(int(root)), _ptr(gamma, f32p),
                                                   C.c_int32(len(gamma)), C.c_float(epsilon)))

    def set_keys(self, nodes, keys):
        """Position keys of single nodes (the game's own getHash() of the states they stand for)."""
        nodes = np.ascontiguousarray(nodes, dtype=np.int32)
        keys = np.ascontiguousarray(keys, dtype=np.uint64)
        assert len(nodes) == len(keys)
        _check(self._lib.omk_forest_set_keys(self._h, _ptr(nodes, i32p), _ptr(keys, C.POINTER(C.c_uint64)),
                                             C.c_int64(len(nodes))))

    def download_redirects(self):
        """Per child slot the node it holds instead of its own, or -1 (slots re-pointed by
        TranspositionTable.select_redirect)."""
        n, _ = self.node_count()
        out = np.empty(n, np.int32)
        _check(self._lib.omk_forest_download_redirects(self._h, C.c_int64(n), _ptr(out, i32p)))
        return out

    def download_structure(self):
        """Returns dict(child_begin, child_count, action) of the current nodes."""
        n, _ = self.node_count()
        out = dict(child_begin=np.empty(n, np.int32), child_count=np.empty(n, np.int32), action=np.empty(n, np.int32))
        _check(self._lib.omk_forest_download_structure(self._h, C.c_int64(n), _ptr(out["child_begin"], i32p),
                                                       _ptr(out["child_count"], i32p), _ptr(out["action"], i32p)))
        return out

    def download(self):
        """Returns dict(N, W, P, VL[, rN, rW]) as numpy arrays."""
        n, _ = self.node_count()
        out = dict(N=np.empty(n, np.int32), W=np.empty(n, np.float32), P=np.empty(n, np.float32),
                   VL=np.empty(n, np.int32))
        if self.has_rave:
            out["rN"] = np.empty(n, np.int32)
            out["rW"] = np.empty(n, np.float32)
        v = _SoaView(n, _ptr(out["N"], i32p), _ptr(out["W"], f32p), _ptr(out["P"], f32p), _ptr(out["VL"], i32p),
                     _ptr(out.get("rN"), i32p), _ptr(out.get("rW"), f32p), i32p(), i32p(), i32p(), u32p(), u64p())
        _check(self._lib.omk_forest_download(self._h, C.byref(v)))
        return out

    # device memory helpers (for callers without their own HIP binding)
    def dev_alloc(self, nbytes):
        p = C.c_void_p()
        _check(self._lib.omk_dev_alloc(self._h, int(nbytes), C.byref(p)))
        return p.value

    def dev_free(self, ptr):
        _check(self._lib.omk_dev_free(self._h, C.c_void_p(ptr)))

    def h2d(self, dptr, arr):
        arr = np.ascontiguousarray(arr)
        _check(self._lib.omk_dev_h2d(self._h, C.c_void_p(dptr), arr.ctypes.data_as(C.c_void_p), arr.nbytes))

    def d2h(self, arr, dptr):
        assert arr.flags["C_CONTIGUOUS"]
        _check(self._lib.omk_dev_d2h(self._h, arr.ctypes.data_as(C.c_void_p), C.c_void_p(dptr), arr.nbytes))

    def dev_copy(self, dst, src, nbytes):
        _check(self._lib.omk_dev_copy(self._h, C.c_void_p(dst), C.c_void_p(src), int(nbytes)))

    # the three node operations over caller-supplied device paths (level-major)
    def apply_vl_paths(self, d_paths, d_len, n, stride, max_len, vl):
        _check(self._lib.omk_apply_vl_paths(self._h, C.c_void_p(d_paths), C.c_void_p(d_len), int(n), int(stride),
                                            int(max_len), int(vl)))

    def revert_vl_paths(self, d_paths, d_len, n, stride, max_len, vl):
        _check(self._lib.omk_revert_vl_paths(self._h, C.c_void_p(d_paths), C.c_void_p(d_len), int(n), int(stride),
                                             int(max_len), int(vl)))

    def backup_paths(self, d_paths, d_len, d_values, n, stride, max_len, vl):
        _check(self._lib.omk_backup_paths(self._h, C.c_void_p(d_paths), C.c_void_p(d_len), C.c_void_p(d_values),
                                          int(n), int(stride), int(max_len), int(vl)))


class Batch:
    """The per-search buffers of executeBatchedTreeSearch: paths, leaves, leaf values."""

    def __init__(self, forest, max_traversals, max_depth):
        self._lib = load_library()
        self.forest = forest
        self.max_traversals = int(max_traversals)
        self.max_depth = int(max_depth)
        self.n = 0
        self._h = C.c_void_p()
        _check(self._lib.omk_batch_create(forest._h, self.max_traversals, self.max_depth, C.byref(self._h)))

    def close(self):
        if self._h:
            self._lib.omk_batch_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_roots(self, roots):
        roots = np.ascontiguousarray(roots, dtype=np.int32)
        _check(self._lib.omk_batch_set_roots(self._h, _ptr(roots, i32p), len(roots)))
        self.n = len(roots)

    def set_values(self, values):
        values = np.ascontiguousarray(values, dtype=np.float32)
        _check(self._lib.omk_batch_set_values(self._h, _ptr(values, f32p), len(values)))

    def select(self, params):
        _check(self._lib.omk_select_batch(self._h, C.byref(params)))

    def backup(self, virtual_loss):
        _check(self._lib.omk_backup_batch(self._h, int(virtual_loss)))

    def backup_rave(self):
        """RAVE statistics of backPropagate for the selected paths and the values set."""
        _check(self._lib.omk_backup_rave_batch(self._h))

    def revert_vl(self, virtual_loss):
        _check(self._lib.omk_revert_vl(self._h, int(virtual_loss)))

    def read(self):
        """Leaf gather: (paths [n, max_depth+1], path_len [n], leaf [n], actions [n, max_depth])."""
        n, D = self.n, self.max_depth
        paths = np.empty((n, D + 1), np.int32)
        plen = np.empty(n, np.int32)
        leaf = np.empty(n, np.int32)
        actions = np.empty((n, D), np.int32)
        _check(self._lib.omk_batch_read(self._h, _ptr(paths, i32p), _ptr(plen, i32p), _ptr(leaf, i32p),
                                        _ptr(actions, i32p)))
        return paths, plen, leaf, actions

    def leaf_keys_dev(self, d_piece_keys, cells, d_player_keys, d_root_keys, d_root_players, d_out):
        _check(self._lib.omk_batch_leaf_keys(self._h, C.c_void_p(d_piece_keys), C.c_int32(int(cells)),
                                             C.c_void_p(d_player_keys), C.c_void_p(d_root_keys),
                                             C.c_void_p(d_root_players), C.c_void_p(d_out)))

    def leaf_keys(self, piece_keys, player_keys, root_keys, root_players):
        """Position key of every selected leaf's state (getHash() of the root state after the path's
        moves): piece_keys [2, cells] and player_keys [2] are the game's Zobrist tables, root_keys /
        root_players [n] the root states' keys and sides to move (0 or 1)."""
        f = self.forest
        pk = np.ascontiguousarray(piece_keys, np.uint64)
        assert pk.ndim == 2 and pk.shape[0] == 2
        pl = np.ascontiguousarray(player_keys, np.uint64)
        rk = np.ascontiguousarray(root_keys, np.uint64)
        rp = np.ascontiguousarray(root_players, np.int32)
        assert len(pl) == 2 and len(rk) == self.n and len(rp) == self.n
        out = np.empty(self.n, np.uint64)
        bufs = [f.dev_alloc(x.nbytes) for x in (pk, pl, rk, rp, out)]
        try:
            for d, x in zip(bufs[:4], (pk, pl, rk, rp)):
                f.h2d(d, x)
            self.leaf_keys_dev(bufs[0], pk.shape[1], bufs[1], bufs[2], bufs[3], bufs[4])
            f.d2h(out, bufs[4])
        finally:
            for d in bufs:
                f.dev_free(d)
        return out

    def expand(self, move_begin, moves, policy=None, action_space=0):
        """Expands the leaves of the last select(): move_begin [n+1] / moves are the legal moves
        every traversal offers for its leaf (empty = terminal), policy None or [n, action_space].
        Returns first_child per traversal (-1 where nothing was added)."""
        mb = np.ascontiguousarray(move_begin, dtype=np.int32)
        mv = np.ascontiguousarray(moves, dtype=np.int32)
        if len(mv) == 0:
            mv = np.zeros(1, np.int32)
        pol = None if policy is None else np.ascontiguousarray(policy, dtype=np.float32)
        first = np.empty(len(mb) - 1, np.int32)
        _check(self._lib.omk_expand_batch(self._h, _ptr(mb, i32p), _ptr(mv, i32p), _ptr(pol, f32p),
                                          C.c_int32(int(action_space)), _ptr(first, i32p)))
        self.forest.node_count()
        return first

    def expand_ex(self, move_begin, moves, policy_begin=None, policy=None, action_space=0, widening=None):
        """expand() with ragged policies (policy_begin [n+1] into policy) and progressive widening
        (widening = (c, k), None = off): see omk_expand_batch_ex."""
        mb = np.ascontiguousarray(move_begin, dtype=np.int32)
        mv = np.ascontiguousarray(moves, dtype=np.int32)
        if len(mv) == 0:
            mv = np.zeros(1, np.int32)
        pb = None if policy_begin is None else np.ascontiguousarray(policy_begin, dtype=np.int32)
        pol = None if policy is None else np.ascontiguousarray(policy, dtype=np.float32).reshape(-1)
        if pol is not None and len(pol) == 0:
            pol = np.zeros(1, np.float32)
        par = _ExpandParams(int(action_space), 0 if widening is None else 1,
                            0.0 if widening is None else float(widening[0]), 0.0 if widening is None else float(widening[1]))
        first = np.empty(len(mb) - 1, np.int32)
        _check(self._lib.omk_expand_batch_ex(self._h, _ptr(mb, i32p), _ptr(mv, i32p), _ptr(pb, i32p), _ptr(pol, f32p),
                                             C.byref(par), _ptr(first, i32p)))
        self.forest.node_count()
        return first

    def truncated(self):
        c = C.c_int32()
        _check(self._lib.omk_batch_truncated(self._h, C.byref(c)))
        return c.value

    def enable_stats(self, on=True):
        """Work statistics of select() (see stats()); off by default, they cost atomics."""
        _check(self._lib.omk_batch_set_stats(self._h, C.c_int32(1 if on else 0)))

    def set_spin_limit(self, polls):
        """Bound of the waits inside the persistent selection kernel (error-path tests)."""
        _check(self._lib.omk_batch_set_spin_limit(self._h, C.c_int32(int(polls))))

    def debug_set_select_count(self, count):
        """Test hook: the number of the select call made last (forward only), to cross the point where the
        call numbers start over without making 2^30 calls."""
        _check(self._lib.omk_debug_set_select_count(self._h, C.c_int32(int(count))))

    def stats(self):
        out = np.zeros(16, np.int32)
        _check(self._lib.omk_batch_stats(self._h, _ptr(out, i32p)))
        keys = ("group_nodes", "water_level_nodes", "settled_by_water_level", "settled_one_by_one",
                "replayed_nodes", "threshold_probes", "single_visitor_steps", "merged_nodes", "t_first_block",
                "t_last_team", "t_last_walker", "walks_in_launch", "narrowed_nodes", "unused_13", "unused_14",
                "sliced_nodes")
        return dict(zip(keys, map(int, out)))

    def enable_trace(self, on=True):
        """The selects that follow record their timeline (see debug_trace())."""
        _check(self._lib.omk_batch_set_trace(self._h, C.c_int32(1 if on else 0)))

    def debug_trace(self, max_entries=1 << 16):
        """Timeline of the last select() after enable_trace(): int64 array [n, 12] of
        (start, end) on the 100 MHz clock, visitors | depth << 32 | kind << 60, node | number << 32 and
        eight words, of which a slice of a heavy node fills two (see omk_debug_trace in the header)."""
        buf = np.zeros((int(max_entries), 12), np.int64)
        n = C.c_int32()
        _check(self._lib.omk_debug_trace(self._h, buf.ctypes.data_as(C.c_void_p), C.c_int32(int(max_entries)),
                                         C.byref(n)))
        return buf[:n.value].copy()

    def device(self):
        d = _BatchDev()
        _check(self._lib.omk_batch_device(self._h, C.byref(d)))
        return d


class TranspositionTable:
    """Open-addressing table in HBM standing in for PHMapTranspositionTable store/lookup."""

    def __init__(self, forest, log2_slots):
        self._lib = load_library()
        self.forest = forest
        self.log2 = int(log2_slots)
        self._h = C.c_void_p()
        _check(self._lib.omk_tt_create(forest._h, self.log2, C.byref(self._h)))

    def close(self):
        if self._h:
            self._lib.omk_tt_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def clear(self):
        _check(self._lib.omk_tt_clear(self._h))

    def insert_dev(self, d_keys, d_nodes, d_depths, n):
        _check(self._lib.omk_tt_insert(self._h, C.c_void_p(d_keys), C.c_void_p(d_nodes), C.c_void_p(d_depths or 0),
                                       int(n)))

    def probe_dev(self, d_keys, n, d_out, min_depth=0):
        _check(self._lib.omk_tt_probe(self._h, C.c_void_p(d_keys), int(n), int(min_depth), C.c_void_p(d_out)))

    def probe_leaves_dev(self, batch, d_out, min_depth=0):
        _check(self._lib.omk_tt_probe_leaves(self._h, batch._h, int(min_depth), C.c_void_p(d_out)))

    def insert(self, keys, nodes, depths=None):
        f = self.forest
        keys = np.ascontiguousarray(keys, np.uint64)
        nodes = np.ascontiguousarray(nodes, np.int32)
        n = len(keys)
        dk, dn = f.dev_alloc(n * 8), f.dev_alloc(n * 4)
        dd = 0
        try:
            f.h2d(dk, keys)
            f.h2d(dn, nodes)
            if depths is not None:
                dd = f.dev_alloc(n * 4)
                f.h2d(dd, np.ascontiguousarray(depths, np.int32))
            self.insert_dev(dk, dn, dd, n)
        finally:
            for p in (dk, dn, dd):
                if p:
                    f.dev_free(p)

    def probe(self, keys, min_depth=0):
        f = self.forest
        keys = np.ascontiguousarray(keys, np.uint64)
        n = len(keys)
        out = np.empty(n, np.int32)
        dk, do = f.dev_alloc(n * 8), f.dev_alloc(n * 4)
        try:
            f.h2d(dk, keys)
            self.probe_dev(dk, n, do, min_depth)
            f.d2h(out, do)
        finally:
            f.dev_free(dk)
            f.dev_free(do)
        return out

    def probe_leaves(self, batch, min_depth=0):
        f = self.forest
        out = np.empty(batch.n, np.int32)
        do = f.dev_alloc(batch.n * 4)
        try:
            self.probe_leaves_dev(batch, do, min_depth)
            f.d2h(out, do)
        finally:
            f.dev_free(do)
        return out

    def store(self, keys, nodes, depths=None):
        """PHMapTranspositionTable::store for a batch; returns (new entries, replacements, duplicates dropped)."""
        f = self.forest
        keys = np.ascontiguousarray(keys, np.uint64)
        nodes = np.ascontiguousarray(nodes, np.int32)
        n = len(keys)
        counts = np.zeros(4, np.int32)
        dk, dn = f.dev_alloc(n * 8), f.dev_alloc(n * 4)
        dd = 0
        try:
            f.h2d(dk, keys)
            f.h2d(dn, nodes)
            if depths is not None:
                dd = f.dev_alloc(n * 4)
                f.h2d(dd, np.ascontiguousarray(depths, np.int32))
            _check(self._lib.omk_tt_store(self._h, C.c_void_p(dk), C.c_void_p(dn), C.c_void_p(dd or 0), C.c_int64(n),
                                          _ptr(counts, i32p)))
        finally:
            for p in (dk, dn, dd):
                if p:
                    f.dev_free(p)
        return tuple(int(x) for x in counts[:3])

    def set_replacement_threshold(self, threshold):
        _check(self._lib.omk_tt_set_replacement_threshold(self._h, C.c_float(threshold)))

    def traverse(self, batch, zobrist=None):
        """The table's part of the traversal loop over the paths of batch's last select(): stores the
        unvisited selected children, looks every step up, reports transpositions.  zobrist: None (the
        forest's per-node keys) or (piece_keys [2, cells], player_keys [2], root_keys [n], root_players [n]).
        Returns (hits [n, max_depth] node or -1, (new entries, replacements, duplicates, transpositions))."""
        f = self.forest
        n, D = batch.n, batch.max_depth
        hits = np.empty((n, D), np.int32)
        counts = np.zeros(4, np.int32)
        bufs = [f.dev_alloc(hits.nbytes)]
        args = [0, 0, 0, 0, 0]
        try:
            if zobrist is not None:
                pk = np.ascontiguousarray(zobrist[0], np.uint64)
                arrs = (pk, np.ascontiguousarray(zobrist[1], np.uint64), np.ascontiguousarray(zobrist[2], np.uint64),
                        np.ascontiguousarray(zobrist[3], np.int32))
                for x in arrs:
                    bufs.append(f.dev_alloc(x.nbytes))
                    f.h2d(bufs[-1], x)
                args = [bufs[1], pk.shape[1], bufs[2], bufs[3], bufs[4]]
            _check(self._lib.omk_tt_traverse(self._h, batch._h, C.c_void_p(args[0]), C.c_int32(int(args[1])),
                                             C.c_void_p(args[2]), C.c_void_p(args[3]), C.c_void_p(args[4]),
                                             C.c_void_p(bufs[0]), _ptr(counts, i32p)))
            f.d2h(hits, bufs[0])
        finally:
            for d in bufs:
                f.dev_free(d)
        return hits, tuple(int(x) for x in counts)

    def select_redirect(self, batch, params, want_moves=True):
        """The traversal loop with the table on, redirects included (omk_tt_select_redirect): a select for
        batch's roots, one traversal after the other, that re-points child slots at transpositions as the
        reference does.  Returns (moves [n, max_depth] recorded at every step, -1 padded, or None;
        (new entries, replacements, lookups that found an entry, redirects, steps))."""
        f = self.forest
        p = params
        counts = np.zeros(5, np.int32)
        n, D = batch.n, batch.max_depth
        stride = int(batch.device().stride)
        d_moves = f.dev_alloc(4 * D * stride) if want_moves else 0
        try:
            _check(self._lib.omk_tt_select_redirect(self._h, batch._h, C.byref(p), C.c_void_p(d_moves),
                                                    _ptr(counts, i32p)))
            moves = None
            if want_moves:
                raw = np.empty((D, stride), np.int32)
                f.d2h(raw, d_moves)
                plen = np.empty(n, np.int32)
                _check(self._lib.omk_batch_read(batch._h, None, _ptr(plen, i32p), None, None))
                moves = np.ascontiguousarray(raw[:, :n].T)
                moves[np.arange(D)[None, :] >= (plen[:, None] - 1)] = -1
        finally:
            if d_moves:
                f.dev_free(d_moves)
        return moves, tuple(int(x) for x in counts)

    def download_meta(self):
        meta = np.empty(1 << self.log2, dtype=TT_META)
        _check(self._lib.omk_tt_download_meta(self._h, meta.ctypes.data_as(C.c_void_p)))
        return meta

    def upload(self, slots):
        slots = np.ascontiguousarray(slots, dtype=TT_SLOT)
        assert len(slots) == 1 << self.log2
        _check(self._lib.omk_tt_upload(self._h, slots.ctypes.data_as(C.c_void_p)))

    def download(self):
        slots = np.empty(1 << self.log2, dtype=TT_SLOT)
        _check(self._lib.omk_tt_download(self._h, slots.ctypes.data_as(C.c_void_p)))
        return slots
