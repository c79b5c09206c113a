"""Randomised parity: forests of random shape and crowd size, selection + backup on the GPU
against the CPU checker (paths, leaves, virtual loss and visit counts bit-exact).  The shapes
are drawn so that every way a crowded node can be settled comes up: runs of one child,
single batches, several batches, slices of heavy nodes, plateaus of RAVE-dominated children,
masked children, pre-existing virtual loss, exact ties, several trees."""
import numpy as np
import pytest

from tests.helpers import random_tree
from tests.test_gpu_scheduler import chain_forest, layered_forest, select_both

pytestmark = pytest.mark.gpu


# (seed 6: its 58th forest once lost a visitor, because the contexts of heavy nodes of a NEW batch were memory an
# earlier batch of the process had left behind, and a context says by the number of the select call, which
# starts again at 1 with every batch, that the contexts of its children are listed)
@pytest.mark.parametrize("seed", [1, 2, 3, 4, 6])
def test_random_forests_and_crowds(seed):
    rng = np.random.default_rng(seed)
    replayed = []
    for case in range(60):
        kind = int(rng.integers(4))
        s = int(rng.integers(1 << 30))
        if kind == 0:
            fan = int(rng.integers(4, 380))
            rave = bool(rng.integers(2))
            plateau = rave and bool(rng.integers(2))
            soa, _ = layered_forest(s, [fan, int(rng.integers(4, 60)), int(rng.integers(4, 8))], rave=rave,
                                    plateau=plateau)
            B = int(rng.integers(100, 9000))
            st = select_both(soa, np.zeros(B, np.int32), 4, rave=rave, steps=2)
        elif kind == 1:
            soa = chain_forest(s, int(rng.integers(3, 30)), int(rng.integers(2, 80)), bool(rng.integers(2)))
            B = int(rng.integers(10, 3000))
            st = select_both(soa, np.zeros(B, np.int32), 40, steps=2)
        elif kind == 2:
            rave = bool(rng.integers(2))
            soa, _ = random_tree(s, n_expand=int(rng.integers(5, 200)), fanout=(1, int(rng.integers(2, 100))),
                                 max_depth=int(rng.integers(2, 9)), rave=rave, mask_frac=float(rng.choice([0, 0.3])),
                                 vl_frac=0.2, tie_frac=0.1, n_max=int(rng.integers(2, 400)))
            B = int(rng.integers(2, 6000))
            st = select_both(soa, np.zeros(B, np.int32), 10, rave=rave, steps=2)
        else:
            soa, roots = layered_forest(s, [int(rng.integers(4, 300)), int(rng.integers(4, 40))],
                                        n_trees=int(rng.integers(1, 5)))
            B = int(rng.integers(1000, 12000))
            tr = np.sort(rng.integers(0, len(roots), B)).astype(np.int32)
            st = select_both(soa, roots[tr], 3, steps=2)
        if st["replayed_nodes"]:
            replayed.append((case, kind, st["replayed_nodes"], st["group_nodes"], st.get("merged_nodes")))
    # a node whose checks fail is replayed one visitor at a time: allowed (the results above are
    # exact either way), but it must stay the exception
    print("replayed:", replayed)
    assert sum(r[2] for r in replayed) <= 3, replayed


@pytest.mark.parametrize("first", [0, 25])
def test_values_that_are_not_finite_with_crowds(first):
    """NaN priors, value sums of -inf, NaN or 3e38, exact ties at zero, virtual loss 0 and 1000, under crowds
    of up to 9000 visitors, with and without RAVE.  (Seed 29: an unvisited child whose value sum is -inf scores
    0 + exploration once and -inf from then on while its RAVE blend stays real, so the reference's first scan
    runs dry in the middle of a node's visitors and the least visited child takes the rest: a node with such a
    child is settled one visitor after the other.)"""
    for seed in range(first, first + 25):
        rng = np.random.default_rng(seed)
        rave = bool(rng.integers(2))
        if rng.random() < 0.5:
            soa, _ = random_tree(int(rng.integers(1 << 30)), n_expand=int(rng.integers(5, 200)),
                                 fanout=(1, int(rng.integers(2, 300))), max_depth=int(rng.integers(2, 8)), rave=rave,
                                 mask_frac=float(rng.choice([0.0, 0.3])), vl_frac=0.2, tie_frac=0.2,
                                 n_max=int(rng.integers(2, 500)))
            D = 9
        else:
            lay = [int(rng.integers(4, 380)), int(rng.integers(4, 30)), int(rng.integers(2, 6))]
            soa, _ = layered_forest(int(rng.integers(1 << 30)), lay, rave=rave)
            D = 4
        n = len(soa["N"])
        soa["P"], soa["W"], soa["N"] = soa["P"].copy(), soa["W"].copy(), soa["N"].copy()
        kind = int(rng.integers(5))
        idx = rng.random(n) < float(rng.choice([0.02, 0.2, 0.9]))
        idx[0] = False
        if kind == 0:
            soa["P"][idx] = np.nan
        elif kind == 1:
            soa["W"][idx] = -np.inf
        elif kind == 2:
            soa["W"][idx] = np.nan
        elif kind == 3:
            soa["P"][idx], soa["N"][idx], soa["W"][idx] = 0.0, 0, 0.0
        else:
            soa["W"][idx] = np.float32(3e38)
        vl = int(rng.choice([0, 0, 1, 3, 1000]))
        B = int(rng.integers(2, 9000))
        select_both(soa, np.zeros(B, np.int32), D, rave=rave, steps=2, vl=vl)


def test_the_widest_fan_out_class_with_crowds():
    """Nodes of 385 to 1024 children (never cut into slices: one wavefront settles them batch after batch), one
    to three trees, up to 12000 visitors."""
    for seed in range(15):
        rng = np.random.default_rng(seed)
        lay = [int(rng.integers(385, 1025)), int(rng.integers(2, 30))]
        if rng.random() < 0.4:
            lay.append(int(rng.integers(2, 6)))
        rave = bool(rng.integers(2))
        plateau = rave and bool(rng.integers(2)) and min(lay) >= 3
        soa, roots = layered_forest(int(rng.integers(1 << 30)), lay, n_trees=int(rng.integers(1, 4)), rave=rave,
                                    plateau=plateau)
        B = int(rng.integers(2, 12000))
        tr = np.sort(rng.integers(0, len(roots), B)).astype(np.int32)
        select_both(soa, roots[tr], len(lay) + 1, rave=rave, steps=2, vl=int(rng.integers(1, 5)))


def test_wide_nodes_with_rave_settled_through_the_children_that_can_be_chosen():
    """With RAVE, a node of more than 64 child slots whose 24 to 1023 visitors split is settled through the few
    children that can be chosen at all, moved to one lane each (the counter says how often).  Forests with the
    statistics of the Go workload (a few children dominate a node) at several sizes of crowd, and random shapes
    of 65 to 380 slots with masks, plateaus and pre-existing virtual loss."""
    from omoknuni_small_amd import synth
    narrowed = 0
    for seed, B in enumerate((2000, 5000, 9000, 16000)):
        soa, roots, meta = synth.generate("c4", seed=40 + seed, nodes_per_tree=600_000)
        st = select_both(soa, synth.traversal_roots(roots, B), int(meta["max_depth"]), rave=True, steps=3,
                         vl=int(meta["virtual_loss"]) if seed % 2 else 1, rave_k=float(meta.get("rave_k", 3000.0)))
        narrowed += st["narrowed_nodes"]
    print("nodes settled that way:", narrowed)
    assert narrowed >= 5, narrowed  # (the full-size Go workload has 20 to 30 such nodes a selection)
    for seed in range(12):
        rng = np.random.default_rng(1000 + seed)
        if seed % 3 == 2:
            soa, _ = random_tree(int(rng.integers(1 << 30)), n_expand=int(rng.integers(20, 120)),
                                 fanout=(65, int(rng.integers(70, 380))), max_depth=int(rng.integers(3, 7)), rave=True,
                                 mask_frac=float(rng.choice([0.0, 0.3])), vl_frac=0.2, tie_frac=0.1,
                                 n_max=int(rng.integers(50, 4000)))
            D = 8
            roots = np.zeros(int(rng.integers(24, 3000)), np.int32)
        else:
            lay = [int(rng.integers(65, 380)), int(rng.integers(65, 200)), int(rng.integers(3, 7))]
            soa, r = layered_forest(int(rng.integers(1 << 30)), lay, n_trees=int(rng.integers(1, 3)), rave=True,
                                    plateau=bool(rng.integers(2)))
            D = 4
            B = int(rng.integers(24, 4000))
            roots = r[np.sort(rng.integers(0, len(r), B))].astype(np.int32)
        select_both(soa, roots, D, rave=True, steps=3, vl=int(rng.integers(1, 4)),
                    rave_k=float(rng.choice([300.0, 1000.0, 3000.0])))


def test_selection_time_widening_with_crowds():
    """omk_select_params::pw (only the ceil(sqrt(N_parent)) children of highest prior take part) on forests
    whose children are stored by descending prior, parents of few and of many visits, crowds up to 12000."""
    import omoknuni_small_amd as omk
    from oracle import ref_cpu as R
    for seed in range(15):
        rng = np.random.default_rng(seed)
        lay = [int(rng.integers(4, 380)), int(rng.integers(4, 40)), int(rng.integers(2, 8))]
        rave = bool(rng.integers(2))
        soa, roots = layered_forest(int(rng.integers(1 << 30)), lay, n_trees=int(rng.integers(1, 4)), rave=rave)
        P = soa["P"].copy()
        for node in np.nonzero(soa["child_count"] > 0)[0]:
            cb, cc = soa["child_begin"][node], soa["child_count"][node]
            P[cb:cb + cc] = np.sort(P[cb:cb + cc])[::-1]
        soa["P"] = P
        soa["N"] = soa["N"].copy()
        small = (rng.random(len(P)) < 0.3) & (soa["child_count"] > 0)
        soa["N"][small] = rng.integers(0, 50, int(small.sum()))
        B, D, vl = int(rng.integers(2, 12000)), 4, int(rng.integers(1, 5))
        troots = roots[np.sort(rng.integers(0, len(roots), B))].astype(np.int32)
        ref = R.RefTree.from_soa(soa)
        rp = R.make_params(c_puct=1.4, virtual_loss=vl, use_rave=rave, rave_k=1000.0, pw=True, max_depth=D)
        f = omk.Forest.from_soa(soa)
        b = omk.Batch(f, B, D)
        b.set_roots(troots)
        sp = omk.SelectParams(c_puct=1.4, virtual_loss=vl, use_rave=rave, rave_k=1000.0, pw=True)
        for step in range(2):
            rpaths, rlen, rleaf, _ = ref.select_batch(troots, rp, near_ties=False)
            b.select(sp)
            gpaths, glen, gleaf, _ = b.read()
            assert (gpaths == rpaths).all() and (glen == rlen).all() and (gleaf == rleaf).all(), (seed, step)
            vals = rng.uniform(-1, 1, B).astype(np.float32)
            ref.backup_batch(rpaths, rlen, vals, vl)
            b.set_values(vals)
            b.backup(vl)
            st = f.download()
            assert (st["N"] == ref.N).all() and (st["VL"] == ref.VL).all(), (seed, step)
            ref.W[:] = st["W"]
        b.close()
        f.close()
