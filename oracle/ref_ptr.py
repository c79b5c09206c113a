"""ctypes wrapper of ref_ptr.cpp: the checker's arithmetic over the reference's node layout
(pointer tree, one cache line per atomic field, include/mcts/mcts_node.h:154-178) and its
OpenMP traversal / backup loops (src/mcts/mcts_engine_batch_tree_simple.cpp:73-185, :276-281).

TEST INFRASTRUCTURE ONLY: used by the benchmark's cpu_baseline leg and by the tests."""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
i32p = C.POINTER(C.c_int32)
f32p = C.POINTER(C.c_float)
u32p = C.POINTER(C.c_uint32)


def build(force=False):
    so = os.path.join(_HERE, "libref_ptr.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libref_ptr.so"])
    return so


def lib():
    global _LIB
    if _LIB is None:
        L = C.CDLL(build())
        L.ref_ptr_create.restype = C.c_void_p
        L.ref_ptr_create.argtypes = [C.c_int64, i32p, f32p, f32p, i32p, i32p, f32p, i32p, i32p, i32p, u32p]
        L.ref_ptr_destroy.argtypes = [C.c_void_p]
        L.ref_ptr_destroy.restype = None
        L.ref_ptr_step.restype = C.c_int
        L.ref_ptr_step.argtypes = [C.c_void_p, i32p, C.c_int32, C.c_float, C.c_int32, C.c_int32, C.c_float, C.c_int32,
                                   C.c_int32, f32p, C.c_int32, i32p, i32p, C.POINTER(C.c_double),
                                   C.POINTER(C.c_double)]
        L.ref_ptr_download.argtypes = [C.c_void_p, i32p, f32p, i32p]
        L.ref_ptr_download.restype = None
        L.ref_ptr_node_bytes.restype = C.c_int64
        _LIB = L
    return _LIB


def _p(a, t):
    return None if a is None else a.ctypes.data_as(t)


class PtrTree:
    """The forest as a tree of heap nodes, built from the same arrays as RefTree.from_soa."""

    def __init__(self, soa):
        g = lambda k, dt: None if soa.get(k) is None else np.ascontiguousarray(soa[k], dtype=dt)
        self.n = len(soa["N"])
        arrs = [g("N", np.int32), g("W", np.float32), g("P", np.float32), g("VL", np.int32), g("rN", np.int32),
                g("rW", np.float32), g("child_begin", np.int32), g("child_count", np.int32), g("action", np.int32)]
        legal = g("legal", np.uint32)
        self._h = lib().ref_ptr_create(self.n, _p(arrs[0], i32p), _p(arrs[1], f32p), _p(arrs[2], f32p),
                                       _p(arrs[3], i32p), _p(arrs[4], i32p), _p(arrs[5], f32p), _p(arrs[6], i32p),
                                       _p(arrs[7], i32p), _p(arrs[8], i32p), _p(legal, u32p))

    def close(self):
        if self._h:
            lib().ref_ptr_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def step(self, roots, values, c_puct=1.4, virtual_loss=3, use_rave=False, rave_k=3000.0, pw=False, max_depth=32,
             threads=1):
        """Traversal loop then backup loop; returns (paths[B][max_depth+1], path_len, select s, backup s)."""
        roots = np.ascontiguousarray(roots, np.int32)
        values = np.ascontiguousarray(values, np.float32)
        B = len(roots)
        paths = np.empty((B, max_depth + 1), np.int32)
        plen = np.empty(B, np.int32)
        s, b = C.c_double(0), C.c_double(0)
        rc = lib().ref_ptr_step(self._h, _p(roots, i32p), B, c_puct, int(virtual_loss), int(bool(use_rave)),
                                float(rave_k), int(bool(pw)), int(max_depth), _p(values, f32p), int(threads),
                                _p(paths, i32p), _p(plen, i32p), C.byref(s), C.byref(b))
        assert rc == 0
        return paths, plen, s.value, b.value

    def download(self):
        N = np.empty(self.n, np.int32)
        W = np.empty(self.n, np.float32)
        VL = np.empty(self.n, np.int32)
        lib().ref_ptr_download(self._h, _p(N, i32p), _p(W, f32p), _p(VL, i32p))
        return dict(N=N, W=W, VL=VL)

    @staticmethod
    def node_bytes():
        return int(lib().ref_ptr_node_bytes())
