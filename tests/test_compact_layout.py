"""The host-side re-layout of a board forest without its empty slots (omk_soa_compact_legal).
On the CPU: the re-laid forest is the same forest (the checker selects the same nodes, through the
id map, with the same move lists, step after step).  On the GPU: the HIP path on the re-laid
forest against the checker on the ORIGINAL layout."""
import numpy as np
import pytest

from oracle import ref_cpu as R
from helpers import random_tree

W_RTOL = 1e-5


def scaled(name, **kw):
    from omoknuni_small_amd import synth
    soa, roots, meta = synth.generate(name, seed=23, **kw)
    return soa, roots, meta, synth


def mapped_paths(paths, plen, new_to_old):
    out = np.full_like(paths, -1)
    on = np.arange(paths.shape[1])[None, :] < plen[:, None]
    out[on] = new_to_old[paths[on]]
    return out


@pytest.mark.parametrize("name,kw,B", [("c0", dict(nodes_per_tree=30_000), 200),
                                       ("c2", dict(n_trees=3, nodes_per_tree=40_000), 48),
                                       ("c4", dict(nodes_per_tree=80_000), 600)])
def test_relaid_forest_is_the_same_forest_for_the_checker(name, kw, B):
    import omoknuni_small_amd as omk
    soa, roots, meta, synth = scaled(name, **kw)
    comp, o2n, n2o = omk.compact_legal(soa)
    n = len(soa["N"])
    bits = np.unpackbits(soa["legal"].view(np.uint8), bitorder="little")[:n].astype(bool)
    assert len(comp["N"]) == int(bits.sum()) and "legal" not in comp
    assert (n2o == np.nonzero(bits)[0]).all()                       # old order kept
    assert (o2n[bits] == np.arange(len(n2o))).all() and (o2n[~bits] == -1).all()
    for k in ("N", "W", "P", "VL", "action") + (("rN", "rW") if "rN" in soa else ()) + (("hash",) if "hash" in soa else ()):
        assert (comp[k] == soa[k][n2o]).all(), k
    # a child range holds exactly the legal children of the old range, in order
    exp = np.nonzero(soa["child_count"][n2o] > 0)[0][:2000]
    for j in exp:
        i = n2o[j]
        kids = np.arange(soa["child_begin"][i], soa["child_begin"][i] + soa["child_count"][i])
        kids = kids[bits[kids]]
        assert comp["child_count"][j] == len(kids)
        if len(kids):
            assert (n2o[comp["child_begin"][j]:comp["child_begin"][j] + len(kids)] == kids).all()
    assert int(comp["child_count"].max()) <= 256 + 64   # what the narrower kernel instantiation needs, roughly

    D, vl = int(meta["max_depth"]), int(meta["virtual_loss"])
    rave, rave_k = bool(meta.get("has_rave")), float(meta.get("rave_k", 3000.0))
    rp = R.make_params(c_puct=meta["c_puct"], virtual_loss=vl, use_rave=rave, rave_k=rave_k, pw=False, max_depth=D)
    troots = synth.traversal_roots(roots, B)
    a, b = R.RefTree.from_soa(soa), R.RefTree.from_soa(comp)
    rng = np.random.default_rng(3)
    for step in range(3):
        pa, la, fa, _ = a.select_batch(troots, rp)
        pb, lb, fb, _ = b.select_batch(o2n[troots], rp)
        assert (la == lb).all() and (mapped_paths(pb, lb, n2o) == pa).all() and (n2o[fb] == fa).all(), step
        assert (a.gather_actions(pa, la) == b.gather_actions(pb, lb)).all()
        values = rng.uniform(-1, 1, B).astype(np.float32)
        a.backup_batch(pa, la, values, vl)
        b.backup_batch(pb, lb, values, vl)
        assert (a.N[n2o] == b.N).all() and (a.VL[n2o] == b.VL).all() and (a.W[n2o] == b.W).all()


def test_relayout_without_an_action_array_and_without_a_mask():
    import omoknuni_small_amd as omk
    soa, roots = random_tree(5, n_expand=60, fanout=(2, 20), mask_frac=0.4, n_roots=2, rave=True)
    slot = np.array(soa["action"])
    del soa["action"]
    comp, o2n, n2o = omk.compact_legal(soa)
    kept_children = np.nonzero(slot[n2o] >= 0)[0]
    assert (comp["action"][kept_children] == slot[n2o][kept_children]).all()   # slot in the parent's range
    assert (comp["action"][o2n[np.asarray(roots)]] == -1).all()
    nomask = {k: v for k, v in soa.items() if k != "legal"}
    same, o2n2, n2o2 = omk.compact_legal(nomask)
    assert (n2o2 == np.arange(len(soa["N"]))).all() and (same["child_begin"][same["child_count"] > 0]
                                                         == soa["child_begin"][soa["child_count"] > 0]).all()
    with pytest.raises(omk.OmkError):
        bad = dict(soa)
        bad["child_count"] = soa["child_count"].copy()
        bad["child_count"][np.asarray(roots)[0]] = len(soa["N"]) + 5
        omk.compact_legal(bad)


@pytest.mark.gpu
@pytest.mark.parametrize("name,kw,B", [("c0", dict(nodes_per_tree=40_000), 3000),
                                       ("c2", dict(n_trees=6, nodes_per_tree=60_000), 96),
                                       ("c4", dict(nodes_per_tree=300_000), 5000),
                                       ("wide", dict(n_trees=512), 512)])
def test_gpu_on_the_relaid_forest_against_the_checker_on_the_original(name, kw, B):
    import omoknuni_small_amd as omk
    soa, roots, meta, synth = scaled(name, **kw)
    comp, o2n, n2o = omk.compact_legal(soa)
    D, vl = int(meta["max_depth"]), int(meta["virtual_loss"])
    rave, rave_k = bool(meta.get("has_rave")), float(meta.get("rave_k", 3000.0))
    troots = synth.traversal_roots(roots, B)
    ref = R.RefTree.from_soa(soa)
    rp = R.make_params(c_puct=meta["c_puct"], virtual_loss=vl, use_rave=rave, rave_k=rave_k, pw=False, max_depth=D)
    forest = omk.Forest.from_soa(comp)
    batch = omk.Batch(forest, B, D)
    batch.set_roots(o2n[troots])
    sp = omk.SelectParams(c_puct=meta["c_puct"], virtual_loss=vl, use_rave=rave, rave_k=rave_k, pw=False)
    rng = np.random.default_rng(5)
    for step in range(3):
        rpaths, rlen, rleaf, near = ref.select_batch(troots, rp)
        batch.select(sp)
        gpaths, glen, gleaf, gact = batch.read()
        assert (glen == rlen).all() and (mapped_paths(gpaths, glen, n2o) == rpaths).all(), step
        assert (n2o[gleaf] == rleaf).all()
        assert (gact == ref.gather_actions(rpaths, rlen)).all()
        values = rng.uniform(-1, 1, B).astype(np.float32)
        ref.backup_batch(rpaths, rlen, values, vl)
        batch.set_values(values)
        batch.backup(vl)
        st = forest.download()
        assert (st["N"] == ref.N[n2o]).all() and (st["VL"] == ref.VL[n2o]).all()
        err = np.abs(st["W"].astype(np.float64) - ref.W[n2o]) / np.maximum(np.abs(ref.W[n2o]), 1.0)
        assert err.max() <= W_RTOL
        # keep both sides on identical floats for the next step (the sums above differ in the last bits)
        ref.W[n2o] = st["W"]
    batch.close()
    forest.close()
