"""Pins the CPU checker to the reference: recorded known answers of the reference node class
and the facts asserted by the reference's own unit tests."""
import struct

import numpy as np
import pytest

from oracle import ref_cpu as R
from tests.helpers import star


def bits(x):
    return struct.pack(">f", float(x)).hex()


def test_kat_select(golden):
    for k in golden["select"]:
        rave = "rave" in k
        t = R.RefTree.from_soa(star(k["Np"], k["children"], rave=rave))
        p = R.make_params(c_puct=k["c"], use_rave=False)
        assert t.select_child(0, p) - 1 == k["plain"], k["id"]
        if rave:
            p = R.make_params(c_puct=k["c"], use_rave=True, rave_k=k["rave_k"])
            assert t.select_child(0, p) - 1 == k["rave"], k["id"]
        if "combined_bits" in k:
            got = [bits(t.combined_value(i + 1, k["rave_k"])) for i in range(len(k["children"]))]
            assert got == k["combined_bits"]


def test_kat_score_bits(golden):
    for k in golden["score_bits"]:
        t = R.RefTree.from_soa(star(k["Np"], [k["child"]]))
        p = R.make_params(c_puct=k["c"])
        s1, s2 = t.child_scores(0, 1, p)
        assert bits(s1) == k["score"]
        assert bits(s2) == k["score"]
        ep = np.float32(k["c"]) * np.sqrt(np.float32(k["Np"]))
        assert bits(ep) == k["exploration_param"]
        n, w, pr, vl = k["child"][:4]
        q = (np.float32(w) - np.float32(vl)) / np.float32(n + vl)
        u = (np.float32(pr) * ep) / (np.float32(1.0) + np.float32(n + vl))
        assert bits(q) == k["exploitation"] and bits(u) == k["exploration"]
        assert bits(np.float32(q + u)) == k["score"]


def test_kat_backup(golden):
    k = golden["backup"][0]
    nd = k["nodes"]
    order = ["root", "a", "b", "c"]
    t = R.RefTree(N=[nd[x][0] for x in order], W=[nd[x][1] for x in order], P=[0, 1, 1, 1], VL=[0] * 4,
                  child_begin=[1, 2, 3, 0], child_count=[1, 1, 1, 0])
    p = R.make_params(virtual_loss=k["virtual_loss"], max_depth=8)
    paths, plen, leaf, _ = t.select_batch([0], p)
    assert list(paths[0, :4]) == [0, 1, 2, 3] and plen[0] == 4 and leaf[0] == 3
    assert list(t.VL) == k["post_select_vl"]
    t.backup_batch(paths, plen, [k["leaf_value"]], k["virtual_loss"])
    for i, x in enumerate(order):
        n, w, vl = k["post_backup"][x]
        assert t.N[i] == n and t.VL[i] == vl
        assert t.W[i] == pytest.approx(w, rel=1e-6)
    # exact: the values are sums of one or two float32 terms
    assert t.W[0] == np.float32(0) + (-np.float32(0.6)) and t.W[1] == np.float32(1) + np.float32(0.6)


def test_kat_vl_probe(golden):
    k = golden["virtual_loss_probe"]
    t = R.RefTree(N=[0], W=[0], P=[0], VL=[k["start"]], child_begin=[0], child_count=[0])
    t.update(0, 0.25)
    assert t.VL[0] == k["after_update"]
    t.remove_vl(0, 3)
    assert t.VL[0] == k["after_remove_3"]


# --- facts asserted by the reference's own unit tests -------------------------------------

def test_ref_child_selection():
    # tests/mcts/mcts_node_test.cpp:237-268
    t = R.RefTree.from_soa(star(0, [[0, 0, .7, 0], [0, 0, .2, 0], [0, 0, .1, 0]]))
    p = R.make_params(c_puct=1.0)
    t.update(0, 0.0)
    assert t.select_child(0, p) == 1
    t.update(1, -1.0)
    assert t.select_child(0, p) != 1


def test_ref_virtual_loss_tiebreak():
    # tests/mcts/mcts_node_test.cpp:271-298 -- equal priors: first child, another after VL, first again
    t = R.RefTree.from_soa(star(0, [[0, 0, 1 / 3, 0]] * 3))
    p = R.make_params(c_puct=1.0)
    first = t.select_child(0, p)
    assert first == 1
    t.add_vl(first, 1)
    assert t.select_child(0, p) != first
    t.remove_vl(first)
    assert t.select_child(0, p) == first


def test_ref_backpropagation():
    # tests/mcts/mcts_node_test.cpp:301-313
    t = R.RefTree(N=[0], W=[0], P=[0], VL=[0], child_begin=[0], child_count=[0])
    t.update(0, 1.0)
    t.update(0, 0.5)
    assert t.N[0] == 2 and t.W[0] / t.N[0] == 0.75


def test_ref_virtual_loss_round_trip_and_stacking():
    # tests/mcts/virtual_loss_test.cpp:42-69 and :160-193
    t = R.RefTree(N=[0], W=[0], P=[.2], VL=[0], child_begin=[0], child_count=[0])
    t.add_vl(0, 1)
    assert t.VL[0] == 1
    t.remove_vl(0, 1)
    assert t.VL[0] == 0
    for want in (1, 2, 3):
        t.add_vl(0, 1)
        assert t.VL[0] == want
    t.remove_vl(0, 3)
    assert t.VL[0] == 0


def test_ref_virtual_loss_ucb_impact():
    # tests/mcts/virtual_loss_test.cpp:195-224
    t = R.RefTree.from_soa(star(0, [[0, 0, .2, 0]] * 5))
    for c in range(1, 6):
        for _ in range(10):
            t.update(c, 0.5)
    t.add_vl(1, 3)
    for _ in range(50):
        t.update(0, 0.5)
    assert t.N[0] == 50 and t.N[1] == 10 and t.W[1] == 5.0
    assert t.select_child(0, R.make_params(c_puct=1.5)) != 1


def test_ref_virtual_loss_edge_cases():
    # tests/mcts/virtual_loss_test.cpp:282-308
    t = R.RefTree(N=[0], W=[0], P=[.2], VL=[0], child_begin=[0], child_count=[0])
    t.add_vl(0, -1)
    assert t.VL[0] == 0
    t.add_vl(0, 0)
    assert t.VL[0] == 0
    t.add_vl(0, 1000)
    assert t.VL[0] == 1000
    t.remove_vl(0, 2000)
    assert t.VL[0] == 0
