"""GPU parity on scaled-down versions of the five benchmark workloads, several search steps
in a row (select -> leaf gather -> backup), against the CPU checker after every phase.
These trees have the benchmark's statistics: a few children with thousands of visits
dominate a node, so hundreds of concurrent traversals crowd the same nodes and the
look-ahead rounds of the selection kernel carry most of the work."""
import numpy as np
import pytest

from oracle import ref_cpu as R

pytestmark = pytest.mark.gpu

W_RTOL = 1e-5

CASES = {
    "c0": dict(nodes_per_tree=40_000, B=64),
    "c0_crowded": dict(config="c0", nodes_per_tree=40_000, B=3000),
    "c1": dict(n_trees=16, nodes_per_tree=12_000, B=16),
    "c1_crowded": dict(config="c1", n_trees=5, nodes_per_tree=12_000, B=777),
    "c2": dict(n_trees=6, nodes_per_tree=60_000, B=96),
    "c3": dict(nodes_per_tree=150_000, B=4096),
    "c4": dict(nodes_per_tree=300_000, B=5000),
    "c4_tiny_vl": dict(config="c4", nodes_per_tree=100_000, B=1500, virtual_loss=1),
}


@pytest.mark.parametrize("case", sorted(CASES))
def test_workload_steps(case):
    import omoknuni_small_amd as omk
    from omoknuni_small_amd import synth

    kw = dict(CASES[case])
    name = kw.pop("config", case)
    B = kw.pop("B")
    soa, roots, meta = synth.generate(name, seed=11, **kw)
    D, vl = int(meta["max_depth"]), int(meta["virtual_loss"])
    rave, pw = bool(meta.get("has_rave")), bool(meta.get("pw"))
    rave_k = float(meta.get("rave_k", 3000.0))
    troots = synth.traversal_roots(roots, B)
    ref = R.RefTree.from_soa(soa)
    rp = R.make_params(c_puct=meta["c_puct"], virtual_loss=vl, use_rave=rave, rave_k=rave_k, pw=pw, max_depth=D)
    forest = omk.Forest.from_soa(soa)
    batch = omk.Batch(forest, B, D)
    batch.set_roots(troots)
    sp = omk.SelectParams(c_puct=meta["c_puct"], virtual_loss=vl, use_rave=rave, rave_k=rave_k, pw=pw)
    rng = np.random.default_rng(5)
    total_near = 0
    for step in range(3):
        rpaths, rlen, rleaf, near = ref.select_batch(troots, rp)
        batch.select(sp)
        gpaths, glen, gleaf, gact = batch.read()
        bad = np.nonzero((gpaths != rpaths).any(axis=1) | (glen != rlen) | (gleaf != rleaf))[0]
        total_near += int((near >= 0).sum())
        assert len(bad) == 0, "step %d: %d of %d paths differ (first %s; %d near-tie traversals flagged)" % (
            step, len(bad), B, bad[:5], int((near >= 0).sum()))
        assert (gact == ref.gather_actions(rpaths, rlen)).all()
        st = forest.download()
        assert (st["VL"] == ref.VL).all(), "virtual loss after select, step %d" % step
        values = rng.uniform(-1, 1, B).astype(np.float32)
        ref.backup_batch(rpaths, rlen, values, vl)
        batch.set_values(values)
        batch.backup(vl)
        st = forest.download()
        assert (st["N"] == ref.N).all() and (st["VL"] == ref.VL).all(), "counters after backup, step %d" % step
        err = np.abs(st["W"].astype(np.float64) - ref.W) / np.maximum(np.abs(ref.W), 1.0)
        assert err.max() <= W_RTOL
        # keep both sides on identical floats for the next step (the sums above differ in the last bits)
        ref.W[:] = st["W"]
    print("near-tie traversals flagged by the checker over 3 steps:", total_near)


def test_lookahead_heavy_star():
    """One node, thousands of visitors, a handful of heavily visited children and many light
    ones: long runs, alternation between dominant children, exact ties between clones."""
    import omoknuni_small_amd as omk
    from tests.helpers import star

    rng = np.random.default_rng(3)
    kids = []
    for i in range(150):
        if i % 17 == 0:
            n = 10000
            w = float(rng.uniform(0.9, 0.99)) * n
        else:
            n = int(rng.integers(0, 6))
            w = float(rng.uniform(-n, n))
        kids.append([n, w, float(rng.uniform(0.001, 0.02)), 0])
    kids[34] = list(kids[17])  # exact clones: every one of their scores ties
    kids[51] = list(kids[17])
    soa = star(200000, kids)
    for vl in (3, 1):
        ref = R.RefTree.from_soa(soa)
        B = 6000
        rp = R.make_params(virtual_loss=vl, max_depth=1)
        rpaths, rlen, rleaf, _ = ref.select_batch(np.zeros(B, np.int32), rp)
        f = omk.Forest.from_soa(soa)
        b = omk.Batch(f, B, 1)
        b.set_roots(np.zeros(B, np.int32))
        b.select(omk.SelectParams(virtual_loss=vl))
        gpaths, glen, gleaf, _ = b.read()
        assert (gleaf == rleaf).all(), "first mismatch at traversal %d" % int(np.nonzero(gleaf != rleaf)[0][0])
        assert (f.download()["VL"] == ref.VL).all()
