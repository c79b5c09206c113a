"""GPU parity of the leaf-key table probes (omk_tt_probe_leaves): after a selection, the position key
of every selected leaf (the forest's per-node `hash` array) is looked up in the open-addressing table.
Checked against the CPU checker's table (ref_tt_probe over hash[leaf of the checker's own selection])
and against a Python dict: hits, misses, the min_depth filter, and traversals without a leaf (-1 after
a selection that gave up)."""
import numpy as np
import pytest

from oracle import ref_cpu as R

pytestmark = pytest.mark.gpu


def _table_of(soa, meta, log2, rng, frac_nodes=0.5):
    """Half of the nodes go into the table (50 % load when log2 matches), with a depth each."""
    n = len(soa["N"])
    n_ins = min(1 << (log2 - 1), int(n * frac_nodes))
    ids = np.sort(rng.choice(n, n_ins, replace=False)).astype(np.int32)
    depths = rng.integers(0, 12, n_ins).astype(np.int32)
    return ids, depths


@pytest.mark.parametrize("nodes,B,log2", [(300_000, 5000, 19), (60_000, 700, 17)])
def test_probe_leaves_matches_checker_and_dict(nodes, B, log2):
    import omoknuni_small_amd as omk
    from omoknuni_small_amd import synth

    soa, roots, meta = synth.generate("c4", seed=23, nodes_per_tree=nodes)
    D, vl = int(meta["max_depth"]), int(meta["virtual_loss"])
    rng = np.random.default_rng(nodes)
    ids, depths = _table_of(soa, meta, log2, rng)
    keys = soa["hash"][ids]
    assert len(np.unique(keys)) == len(keys), "the generator's position keys are distinct"

    forest = omk.Forest.from_soa(soa)
    tt = omk.TranspositionTable(forest, log2)
    tt.insert(keys, ids, depths)
    ref_tt = R.RefTT(log2)
    for k, v, d in zip(keys, ids, depths):
        assert ref_tt.insert(k, v, d) == 0
    table = {int(k): (int(v), int(d)) for k, v, d in zip(keys, ids, depths)}

    troots = synth.traversal_roots(roots, B)
    ref = R.RefTree.from_soa(soa)
    rp = R.make_params(c_puct=meta["c_puct"], virtual_loss=vl, use_rave=True, rave_k=float(meta["rave_k"]), max_depth=D)
    batch = omk.Batch(forest, B, D)
    batch.set_roots(troots)
    sp = omk.SelectParams(c_puct=meta["c_puct"], virtual_loss=vl, use_rave=True, rave_k=float(meta["rave_k"]))
    vals = rng.uniform(-1, 1, B).astype(np.float32)
    hits_seen = misses_seen = 0
    for step in range(2):
        rpaths, rlen, rleaf, _ = ref.select_batch(troots, rp)
        batch.select(sp)
        _, _, gleaf, _ = batch.read()
        assert (gleaf == rleaf).all()
        for min_depth in (0, 6, 100):
            got = tt.probe_leaves(batch, min_depth)
            want, n_hits = ref_tt.probe(soa["hash"][rleaf], min_depth)
            assert (got == want).all(), "step %d min_depth %d: first difference at traversal %d" % (
                step, min_depth, int(np.nonzero(got != want)[0][0]))
            by_dict = np.array([table[int(k)][0] if int(k) in table and table[int(k)][1] >= min_depth else -1
                                for k in soa["hash"][rleaf]], np.int32)
            assert (got == by_dict).all()
            if min_depth == 0:
                hits_seen += n_hits
                misses_seen += B - n_hits
            if min_depth == 100:
                assert (got == -1).all()
        ref.backup_batch(rpaths, rlen, vals, vl)
        batch.set_values(vals)
        batch.backup(vl)
        ref.W[:] = forest.download()["W"]
    assert hits_seen > 0 and misses_seen > 0, (hits_seen, misses_seen)


def test_probe_leaves_of_an_incomplete_selection():
    """A selection that gives up (spin limit 0) leaves traversals without a leaf (-1): they find
    nothing, whatever the table holds, and the kernel indexes the key array with no such id."""
    import omoknuni_small_amd as omk
    from omoknuni_small_amd import synth

    soa, roots, meta = synth.generate("c4", seed=5, nodes_per_tree=50_000)
    D, vl, B, log2 = int(meta["max_depth"]), 3, 3000, 16
    forest = omk.Forest.from_soa(soa)
    tt = omk.TranspositionTable(forest, log2)
    ids = np.arange(0, 30_000, dtype=np.int32)
    tt.insert(soa["hash"][ids], ids)
    ref_tt = R.RefTT(log2)
    for k, v in zip(soa["hash"][ids], ids):
        ref_tt.insert(k, v, 0)
    batch = omk.Batch(forest, B, D)
    batch.set_roots(synth.traversal_roots(roots, B))
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=vl, use_rave=True, rave_k=1000.0)
    batch.set_spin_limit(0)
    batch.select(sp)
    with pytest.raises(omk.OmkError):
        batch.read()
    dev = batch.device()
    leaf = np.empty(B, np.int32)
    forest.d2h(leaf, dev.d_leaf)
    assert (leaf == -1).any(), "the forced give-up left every traversal with a leaf: nothing tested"
    got = tt.probe_leaves(batch)
    want = np.full(B, -1, np.int32)
    have = leaf >= 0
    want[have] = ref_tt.probe(soa["hash"][leaf[have]])[0]
    assert (got == want).all()
    # the batch and the table work again afterwards
    batch.set_spin_limit(1 << 22)
    forest.upload(soa)
    ref = R.RefTree.from_soa(soa)
    rp = R.make_params(c_puct=1.4, virtual_loss=vl, use_rave=True, rave_k=1000.0, max_depth=D)
    _, _, rleaf, _ = ref.select_batch(synth.traversal_roots(roots, B), rp)
    batch.select(sp)
    _, _, gleaf, _ = batch.read()
    assert (gleaf == rleaf).all()
    assert (tt.probe_leaves(batch) == ref_tt.probe(soa["hash"][rleaf])[0]).all()


def test_probe_leaves_needs_keys_and_a_selection():
    import omoknuni_small_amd as omk
    from omoknuni_small_amd import synth

    soa, roots, meta = synth.generate("c0", seed=2, nodes_per_tree=5000)
    forest = omk.Forest.from_soa(soa)
    tt = omk.TranspositionTable(forest, 10)
    batch = omk.Batch(forest, 8, 12)
    batch.set_roots(synth.traversal_roots(roots, 8))
    with pytest.raises(omk.OmkError) as e:
        tt.probe_leaves(batch)
    assert e.value.code == -6  # no selection yet
    batch.select(omk.SelectParams())
    with pytest.raises(omk.OmkError) as e:
        tt.probe_leaves(batch)
    assert e.value.code == -6  # the forest holds no position keys
