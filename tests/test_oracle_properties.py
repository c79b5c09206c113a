"""Pins what the reference's fixtures leave open with facts the arithmetic itself fixes:
closed forms, invariants, and brute force on small inputs.  Each check is chosen so that a
plausible slip (dropped term, wrong sign, off-by-one index, wrong tie rule) fails it."""
import math

import numpy as np
import pytest

from oracle import ref_cpu as R
from tests.helpers import random_tree, star

L = R.lib


def test_ceil_sqrt_exhaustive_and_extremes():
    for n in range(0, 70000):
        k = L().ref_ceil_sqrt(n)
        assert k >= 1 and k * k >= n and (k == 1 or (k - 1) * (k - 1) < n), n
    for n in (2**31 - 1, 46340**2, 46340**2 + 1, 46340**2 - 1):
        k = L().ref_ceil_sqrt(n)
        assert k * k >= n and (k - 1) * (k - 1) < n


def test_parent_without_visits_picks_best_mean_and_lowest_index_on_ties():
    # N_parent = 0 kills the exploration term: argmax of W/N, unvisited children count as 0
    t = R.RefTree.from_soa(star(0, [[4, -1.0, .9, 0], [2, 1.0, .01, 0], [0, 0, .5, 0], [2, 1.0, .3, 0]]))
    assert t.select_child(0, R.make_params()) == 2  # children 1 and 3 tie at 0.5: lowest index
    t = R.RefTree.from_soa(star(0, [[0, 0, .1, 0]] * 7))
    assert t.select_child(0, R.make_params()) == 1  # all zero: strict '>' keeps the first


def test_brute_force_double_precision_agrees_outside_near_ties():
    rng = np.random.default_rng(1)
    disagreements = 0
    for trial in range(400):
        k = int(rng.integers(1, 40))
        n = rng.integers(0, 60, k)
        w = np.where(n > 0, rng.uniform(-1, 1, k) * n, 0).astype(np.float32)
        p = rng.dirichlet(np.ones(k)).astype(np.float32)
        vl = rng.integers(0, 4, k) * 3
        Np = int(n.sum() + 1)
        c = float(rng.uniform(0.1, 3))
        t = R.RefTree.from_soa(star(Np, np.stack([n, w, p, vl], 1)))
        got, info = t.select_child(0, R.make_params(c_puct=c), with_info=True)
        ev = (n + vl).astype(np.float64)
        q = np.where(ev > 0, (w.astype(np.float64) - vl) / np.maximum(ev, 1), 0.0)
        u = p.astype(np.float64) * (np.float64(np.float32(c)) * math.sqrt(Np)) / (1.0 + ev)
        want = int(np.argmax(q + u))
        if got - 1 != want:
            disagreements += 1
            assert info["near_tie"], (trial, got - 1, want, info)
    assert disagreements <= 8


def test_score_responds_to_each_term_in_the_right_direction():
    base = [[10, 3.0, .2, 0], [10, 3.0, .2, 0]]
    p = R.make_params(c_puct=1.4)

    def pick(mod):
        kids = [list(base[0]), list(base[1])]
        mod(kids[1])
        return R.RefTree.from_soa(star(50, kids)).select_child(0, p) - 1

    assert pick(lambda k: None) == 0                      # exact tie: first
    assert pick(lambda k: k.__setitem__(1, 3.5)) == 1     # more value wins
    assert pick(lambda k: k.__setitem__(2, .25)) == 1     # more prior wins
    assert pick(lambda k: k.__setitem__(3, -1)) == 1      # negative virtual loss would help
    kids = [[10, 3.0, .2, 3], [10, 3.0, .2, 0]]
    assert R.RefTree.from_soa(star(50, kids)).select_child(0, p) - 1 == 1  # virtual loss hurts
    # the exploration term grows with the parent's visits: a high-prior unvisited child overtakes
    kids = [[50, 30.0, .1, 0], [0, 0.0, .9, 0]]
    assert R.RefTree.from_soa(star(0, kids)).select_child(0, p) - 1 == 0
    assert R.RefTree.from_soa(star(400, kids)).select_child(0, p) - 1 == 1


def test_exploration_uses_raw_parent_visits_not_virtual_loss():
    soa = star(9, [[1, 0.0, .5, 0], [1, 0.05, .5, 0]])
    a = R.RefTree.from_soa(soa)
    soa["VL"][0] = 1000  # the parent's own virtual loss plays no role
    b = R.RefTree.from_soa(soa)
    p = R.make_params()
    assert a.child_scores(0, 1, p) == b.child_scores(0, 1, p)
    s1, _ = a.child_scores(0, 1, p)
    assert s1 == np.float32(0.0) + np.float32(np.float32(.5) * np.float32(np.float32(1.4) * np.float32(3.0))) / np.float32(2.0)


def test_combined_value_closed_forms():
    def cv(n, w, rn, rw, k):
        t = R.RefTree(N=[n], W=[w], P=[0], VL=[0], child_begin=[0], child_count=[0], rN=[rn], rW=[rw])
        return float(t.combined_value(0, k))

    assert cv(0, 0, 0, 0, 1000) == 0.0
    assert cv(0, 0, 8, 4.0, 1000) == 0.5                       # N = 0: beta = 1, pure RAVE mean
    beta = np.sqrt(np.float32(1000) / np.float32(3 * 20 + 1000))
    assert cv(20, 10.0, 0, 0.0, 1000) == float(np.float32(np.float32(1) - beta) * np.float32(0.5))  # no RAVE data
    assert abs(cv(20, 10.0, 50, -50.0, 1e-12) - 0.5) < 1e-6    # k -> 0: plain mean
    assert abs(cv(20, 10.0, 50, -50.0, 1e12) - (-1.0)) < 1e-4  # k -> inf: RAVE mean
    # virtual loss is ignored by the blend
    t = R.RefTree(N=[20], W=[10], P=[0], VL=[30], child_begin=[0], child_count=[0], rN=[5], rW=[1])
    u = R.RefTree(N=[20], W=[10], P=[0], VL=[0], child_begin=[0], child_count=[0], rN=[5], rW=[1])
    assert t.combined_value(0, 1000) == u.combined_value(0, 1000)


def test_rave_selection_is_first_max_over_plain_then_blended_scores():
    rng = np.random.default_rng(2)
    for _ in range(300):
        k = int(rng.integers(2, 12))
        n = rng.integers(0, 30, k)
        w = np.where(n > 0, rng.uniform(-1, 1, k) * n, 0)
        rn = rng.integers(0, 30, k)
        rw = np.where(rn > 0, rng.uniform(-1, 1, k) * rn, 0)
        kids = np.stack([n, w, rng.dirichlet(np.ones(k)), rng.integers(0, 2, k) * 3, rn, rw], 1)
        t = R.RefTree.from_soa(star(int(n.sum()) + 1, kids, rave=True))
        p = R.make_params(use_rave=True, rave_k=500.0)
        s = [t.child_scores(0, i + 1, p) for i in range(k)]
        seq = [x[0] for x in s] + [x[1] for x in s]
        best = -np.inf
        arg = -1
        for pos, v in enumerate(seq):
            if v > best:
                best, arg = v, pos
        assert t.select_child(0, p) - 1 == arg % k
        # without RAVE the second scan can never change the winner
        q = R.make_params(use_rave=False)
        s0 = [t.child_scores(0, i + 1, q) for i in range(k)]
        assert all(a == b for a, b in s0)


def test_virtual_loss_counter_closed_form():
    """m backups of a node: VL -> max(0, x - (a+1) m) for a > 0, and x > 0 ? max(0, x - m) : x for
    a <= 0; m reverts: max(0, x - a m).  Derived from the three node operations, order-free."""
    rng = np.random.default_rng(3)
    for _ in range(500):
        x = int(rng.integers(-5, 40))
        a = int(rng.integers(-1, 6))
        m = int(rng.integers(0, 9))
        t = R.RefTree(N=[0], W=[0], P=[0], VL=[x], child_begin=[0], child_count=[0])
        for _ in range(m):
            t.update(0, 0.25)
            t.remove_vl(0, a)
        want = max(0, x - (a + 1) * m) if a > 0 else (max(0, x - m) if x > 0 else x)
        if m == 0:
            want = x
        assert t.VL[0] == want, (x, a, m)
        assert t.N[0] == m
        t = R.RefTree(N=[0], W=[0], P=[0], VL=[x], child_begin=[0], child_count=[0])
        for _ in range(m):
            t.remove_vl(0, a)
        want = x if (a <= 0 or m == 0) else max(0, x - a * m)
        assert t.VL[0] == want


def test_backup_sign_alternates_from_the_leaf():
    n = 7
    t = R.RefTree(N=[0] * n, W=[0] * n, P=[1] * n, VL=[0] * n, child_begin=list(range(1, n)) + [0],
                  child_count=[1] * (n - 1) + [0])
    paths, plen, leaf, _ = t.select_batch([0], R.make_params(virtual_loss=3, max_depth=10))
    assert plen[0] == n and leaf[0] == n - 1
    assert list(t.VL) == [0] + [3] * (n - 1)           # the root never receives virtual loss
    v = np.float32(0.37)
    t.backup_batch(paths, plen, [v], 3)
    for i in range(n):
        j = n - 1 - i                                   # distance from the leaf
        assert t.W[i] == (v if j % 2 == 0 else -v)
        assert t.N[i] == 1 and t.VL[i] == 0
    assert abs(float(t.W.sum()) - float(v)) < 1e-7     # odd length: one +v is left over


def test_traversal_invariants_on_random_forests():
    for seed in range(5):
        soa, roots = random_tree(100 + seed, n_expand=80, fanout=(1, 30), max_depth=7, n_roots=3, mask_frac=0.3,
                                 vl_frac=0.1)
        t = R.RefTree.from_soa(soa)
        B = np.array([roots[i % 3] for i in range(50)], np.int32)
        p = R.make_params(max_depth=9)
        vl0 = t.VL.copy()
        paths, plen, leaf, _ = t.select_batch(B, p)
        parent = np.full(t.n, -1)
        for v in range(t.n):
            cb, cc = soa["child_begin"][v], soa["child_count"][v]
            parent[cb:cb + cc] = v
        bits = np.unpackbits(soa["legal"].view(np.uint8), bitorder="little")
        counts = np.zeros(t.n, np.int64)
        for i in range(len(B)):
            assert paths[i, 0] == B[i] and leaf[i] == paths[i, plen[i] - 1]
            assert (paths[i, plen[i]:] == -1).all()
            for d in range(1, plen[i]):
                assert parent[paths[i, d]] == paths[i, d - 1]
                assert bits[paths[i, d]] == 1            # never an empty slot
                counts[paths[i, d]] += 1
            assert soa["child_count"][leaf[i]] == 0 or plen[i] == p.max_depth + 1
        assert (t.VL == vl0 + 3 * counts).all()          # +virtual_loss per selection, roots untouched
        acts = t.gather_actions(paths, plen)
        for i in range(len(B)):
            for d in range(1, plen[i]):
                assert acts[i, d - 1] == soa["action"][paths[i, d]]
            assert (acts[i, plen[i] - 1:] == -1).all()


def test_progressive_widening_eligibility():
    rng = np.random.default_rng(4)
    for _ in range(200):
        k = int(rng.integers(1, 30))
        n = rng.integers(0, 20, k)
        w = np.where(n > 0, rng.uniform(-1, 1, k) * n, 0)
        pr = rng.dirichlet(np.ones(k))
        if rng.random() < 0.3:
            pr[int(rng.integers(k))] = pr[0]            # equal priors: the lower index ranks first
        Np = int(rng.integers(0, 200))
        kids = np.stack([n, w, pr, np.zeros(k)], 1)
        t = R.RefTree.from_soa(star(Np, kids))
        pw = R.make_params(pw=True)
        got = t.select_child(0, pw) - 1
        lim = max(1, math.ceil(math.sqrt(Np))) if Np > 0 else 1
        assert lim * lim >= Np
        prf = kids[:, 2].astype(np.float32)
        order = sorted(range(k), key=lambda i: (-prf[i], i))
        elig = sorted(order[:lim])
        assert got in elig
        # same answer as plain selection over a tree that only has the eligible children
        sub = R.RefTree.from_soa(star(Np, kids[elig]))
        assert elig[sub.select_child(0, R.make_params()) - 1] == got
        if lim >= k:
            assert got == t.select_child(0, R.make_params()) - 1
        # storing the children by descending prior (what the device path requires) changes nothing
        perm = np.array(order)
        ts = R.RefTree.from_soa(star(Np, kids[perm]))
        assert perm[ts.select_child(0, pw) - 1] == got


def test_transposition_table_against_dict_and_limits():
    rng = np.random.default_rng(5)
    tt = R.RefTT(8)
    table = {}
    keys = [int(x) for x in rng.integers(0, 2**63, 200, dtype=np.uint64)]
    keys += [i << 56 for i in range(1, 30)]              # colliding home slots
    for i, k in enumerate(keys):
        rc = tt.insert(k, i, i % 5)
        assert rc == (1 if k in table else 0)
        table.setdefault(k, (i, i % 5))
    assert tt.insert(2**64 - 1, 1, 0) == -2              # the empty marker is not a key
    probe = np.array(keys[:50] + [int(x) for x in rng.integers(0, 2**63, 100, dtype=np.uint64)], np.uint64)
    for md in (0, 2, 4):
        out, hits = tt.probe(probe, md)
        want = [table[int(k)][0] if int(k) in table and table[int(k)][1] >= md else -1 for k in probe]
        assert list(out) == want and hits == sum(1 for x in want if x >= 0)
    full = R.RefTT(4)
    for i in range(16):
        assert full.insert(1000 + i, i) == 0
    assert full.insert(5, 5) == -1                       # table full
    out, _ = full.probe(np.array([5, 1003], np.uint64))
    assert list(out) == [-1, 3]
