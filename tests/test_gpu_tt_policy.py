"""GPU parity of the transposition table's store with the replacement policy, of the time stamps of
its lookups and of the table's part of the traversal loop (omk_tt_store, omk_tt_probe,
omk_tt_traverse) against the CPU checker: slots and the policy's per-entry data bit for bit, the
reported transpositions identical."""
import numpy as np
import pytest

from oracle import ref_cpu as R
from tests.helpers import board_forest, random_tree

pytestmark = pytest.mark.gpu


def same_tables(tt, ref_tt, what):
    """The two tables hold the same entries (which slot of a probe chain a key landed in depends on the
    order colliding keys arrived in, and the device takes a call's entries in no order)."""
    dev, meta = tt.download(), tt.download_meta()
    empty = np.uint64(0xFFFFFFFFFFFFFFFF)
    du, ru = dev["key"] != empty, ref_tt.slots["key"] != empty
    assert int(du.sum()) == int(ru.sum()), what
    do, ro = np.argsort(dev["key"][du]), np.argsort(ref_tt.slots["key"][ru])
    for k in ("key", "node", "depth"):
        assert (dev[k][du][do] == ref_tt.slots[k][ru][ro]).all(), "%s: %s" % (what, k)
    assert (meta["visits"][du][do] == ref_tt.meta["visits"][ru][ro]).all(), what
    assert meta["value"][du][do].tobytes() == ref_tt.meta["value"][ru][ro].tobytes(), what
    assert (meta["last_access"][du][do] == ref_tt.meta["last_access"][ru][ro]).all(), what


def test_store_with_replacement_policy_and_lookup_stamps():
    import omoknuni_small_amd as omk
    soa, roots = random_tree(90, n_expand=300, fanout=(2, 12), max_depth=7, n_max=60, zero_frac=0.35)
    n = len(soa["N"])
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa)
    log2 = 11
    tt, ref_tt = omk.TranspositionTable(f, log2), R.RefTT(log2)
    rng = np.random.default_rng(3)
    key_pool = rng.integers(1, 2**63, 900, dtype=np.uint64)
    key_pool[:40] = (np.arange(40, dtype=np.uint64) << np.uint64(53)) | np.uint64(5)   # shared home slots
    total = np.zeros(3, np.int64)
    for call in range(10):
        k = 250
        keys = key_pool[rng.permutation(len(key_pool))[:k]].copy()
        keys[200:] = keys[:50]                                   # the same key several times in one call
        nodes = rng.integers(0, n, k).astype(np.int32)
        nodes[rng.random(k) < 0.05] = -1                         # entries to skip
        depths = rng.integers(0, 30, k).astype(np.int32)
        got = tt.store(keys, nodes, depths)
        want = ref_tt.store(ref, keys, nodes, depths)
        assert got == want, "call %d" % call
        total += got
        same_tables(tt, ref_tt, "after store %d" % call)
        probe = np.concatenate([keys[:120], rng.integers(1, 2**63, 60, dtype=np.uint64)])
        for min_depth in (0, 12):
            assert (tt.probe(probe, min_depth) == ref_tt.lookup(probe, min_depth)[0]).all()
        same_tables(tt, ref_tt, "after lookups %d" % call)
        # a search step moves the statistics the next store reads
        vals = rng.uniform(-1, 1, 64).astype(np.float32)
        b = omk.Batch(f, 64, 7)
        b.set_roots(np.zeros(64, np.int32))
        b.select(omk.SelectParams())
        rp, rl, _, _ = ref.select_batch(np.zeros(64, np.int32), R.make_params(max_depth=7))
        b.set_values(vals)
        b.backup(3)
        ref.backup_batch(rp, rl, vals, 3)
        ref.W[:] = f.download()["W"]
    assert total[0] > 300 and total[1] > 20 and total[2] > 100, total    # new, replaced, duplicates all occurred


@pytest.mark.parametrize("mode", ["node_keys", "zobrist"])
def test_traversal_part_of_the_table(mode):
    import omoknuni_small_amd as omk
    cells = 81
    soa, roots, boards, players = board_forest(31, cells=cells, root_stones=8, n_expand=220, fanout=(2, 9), max_depth=6,
                                               n_roots=3, n_max=40, zero_frac=0.5)
    n = len(soa["N"])
    rng = np.random.default_rng(6)
    piece, player = R.zobrist_tables(9, 2, 2, 1234)
    if mode == "node_keys":
        # a game with captures keeps a key per node; transpositions = nodes that share one
        soa["hash"] = rng.integers(1, 2**63, n, dtype=np.uint64)
        twins = rng.permutation(n)[:200]
        soa["hash"][twins[:100]] = soa["hash"][twins[100:]]
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa)
    B, D, vl = 600, 7, 3
    b = omk.Batch(f, B, D)
    troots = roots[np.arange(B) % len(roots)].astype(np.int32)
    b.set_roots(troots)
    sp, rp = omk.SelectParams(virtual_loss=vl), R.make_params(virtual_loss=vl, max_depth=D)
    log2 = 14
    tt, ref_tt = omk.TranspositionTable(f, log2), R.RefTT(log2)
    ri = np.arange(B) % len(roots)
    root_keys = np.array([R.position_key(boards[i], piece, player, players[i]) for i in ri], np.uint64)
    reported = stored = 0
    for step in range(6):
        rpaths, rlen, rleaf, _ = ref.select_batch(troots, rp)
        b.select(sp)
        gpaths, glen, _, _ = b.read()
        assert (gpaths == rpaths).all()
        if mode == "node_keys":
            step_keys = soa["hash"][np.maximum(rpaths[:, 1:], 0)]
            ghits, gcounts = tt.traverse(b)
        else:
            step_keys = np.zeros((B, D), np.uint64)
            for d in range(1, D + 1):                             # key of the state after d moves of every path
                k, bad = R.leaf_keys(ref, rpaths, np.minimum(rlen, d + 1), boards[ri], players[ri], piece, player)
                assert bad == 0
                step_keys[:, d - 1] = k
            ghits, gcounts = tt.traverse(b, zobrist=(piece, player, root_keys, (players[ri] - 1).astype(np.int32)))
        rhits, rcounts = ref_tt.traverse(ref, rpaths, rlen, step_keys)
        assert gcounts == rcounts, "step %d" % step
        assert (ghits == rhits).all(), "step %d" % step
        same_tables(tt, ref_tt, "step %d" % step)
        reported += gcounts[3]
        stored += gcounts[0]
        vals = rng.uniform(-1, 1, B).astype(np.float32)
        b.set_values(vals)
        b.backup(vl)
        ref.backup_batch(rpaths, rlen, vals, vl)
        ref.W[:] = f.download()["W"]
    assert stored > 50
    if mode == "node_keys":
        assert reported > 0, "no transposition was ever reported: nothing tested"


def test_keys_set_node_by_node_from_the_game():
    """omk_forest_set_keys: a forest uploaded without position keys gets them node by node, as the host
    learns them from the states it replays (IGameState::getHash); nodes without a key are neither stored
    nor found, nodes added by an expansion start without one, an id outside the forest is refused."""
    import omoknuni_small_amd as omk
    soa, roots, boards, players = board_forest(41, cells=81, root_stones=6, n_expand=200, fanout=(2, 8), max_depth=6,
                                               n_roots=2, n_max=30, zero_frac=0.5)
    n = len(soa["N"])
    assert "hash" not in soa
    rng = np.random.default_rng(8)
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa, capacity=n + 64)
    B, D, vl = 400, 7, 3
    b = omk.Batch(f, B, D)
    troots = roots[np.arange(B) % len(roots)].astype(np.int32)
    b.set_roots(troots)
    sp, rp = omk.SelectParams(virtual_loss=vl), R.make_params(virtual_loss=vl, max_depth=D)
    tt, ref_tt = omk.TranspositionTable(f, 13), R.RefTT(13)
    no_key = np.uint64(0xFFFFFFFFFFFFFFFF)
    keys = np.full(n + 64, no_key, np.uint64)
    pool = rng.integers(1, 2**63, 150, dtype=np.uint64)    # fewer keys than nodes: some positions are shared
    stored = reported = 0
    for step in range(5):
        rpaths, rlen, rleaf, _ = ref.select_batch(troots, rp)
        b.select(sp)
        gpaths, glen, gleaf, _ = b.read()
        assert (gpaths == rpaths).all()
        # the host has just replayed the states of these leaves: it knows their keys now
        leaves = np.unique(rleaf)
        new = leaves[keys[leaves] == no_key]
        keys[new] = pool[rng.integers(0, len(pool), len(new))]
        f.set_keys(new, keys[new])
        step_keys = keys[np.maximum(rpaths[:, 1:], 0)]
        ghits, gcounts = tt.traverse(b)
        rhits, rcounts = ref_tt.traverse(ref, rpaths, rlen, step_keys)
        assert gcounts == rcounts and (ghits == rhits).all(), "step %d" % step
        same_tables(tt, ref_tt, "step %d" % step)
        stored += gcounts[0]
        reported += gcounts[3]
        vals = rng.uniform(-1, 1, B).astype(np.float32)
        b.set_values(vals)
        b.backup(vl)
        ref.backup_batch(rpaths, rlen, vals, vl)
        ref.W[:] = f.download()["W"]
    assert stored > 20 and reported > 0, (stored, reported)
    # the leaves' own lookups go by the same keys
    got = tt.probe_leaves(b)
    want, _ = ref_tt.lookup(keys[rleaf])
    assert (got == want).all()
    with pytest.raises(omk.OmkError) as e:
        f.set_keys(np.array([0, n + 1000], np.int32), np.array([5, 6], np.uint64))
    assert e.value.code == -1, e.value       # OMK_ERR_INVALID: the id outside the forest was skipped, the other one set


def test_entries_die_with_the_tree_they_point_into():
    """Entries hold node ids.  A compaction renumbers the nodes and an upload of another tree replaces
    them: whatever was stored before is then what an expired weak pointer is in the reference's table
    (PHMapTranspositionTable::lookup erases it, src/mcts/phmap_transposition_table.cpp:100-108) and must
    neither be found nor stand in the way of a new entry under the same key."""
    import omoknuni_small_amd as omk
    soa, roots = random_tree(91, n_expand=200, fanout=(2, 10), max_depth=6, n_max=40, zero_frac=0.2)
    n = len(soa["N"])
    f = omk.Forest.from_soa(soa, capacity=n)
    tt = omk.TranspositionTable(f, 10)
    rng = np.random.default_rng(5)
    keys = rng.integers(1, 2**63, 300, dtype=np.uint64)
    nodes = rng.integers(0, n, 300).astype(np.int32)
    depths = rng.integers(0, 9, 300).astype(np.int32)
    assert tt.store(keys, nodes, depths)[0] == 300
    assert (tt.probe(keys, 0) == nodes).all()
    # the same statistics again: ids keep their meaning, the entries stay
    f.upload(soa)
    assert (tt.probe(keys, 0) == nodes).all()
    # a compaction below a child of the root renumbers the nodes
    child = int(soa["child_begin"][0])
    n_after = len(f.compact(child))
    assert n_after < n
    assert (tt.probe(keys, 0) == -1).all()
    new_nodes = rng.integers(0, n_after, 300).astype(np.int32)
    got = tt.store(keys, new_nodes, depths)
    assert got[0] == 300 and got[1] == 0, got          # all new: nothing old to replace
    assert (tt.probe(keys, 0) == new_nodes).all()
    # another tree in the same forest: again nothing is left
    f.upload(tiny_tree(50))
    assert (tt.probe(keys, 0) == -1).all()


def tiny_tree(n):
    """A root with n - 1 leaf children."""
    z = np.zeros(n, np.int32)
    cb, cc = z.copy(), z.copy()
    cb[0], cc[0] = 1, n - 1
    return dict(N=z.copy(), W=np.zeros(n, np.float32), P=np.full(n, 1.0 / n, np.float32), VL=z.copy(),
                child_begin=cb, child_count=cc)
