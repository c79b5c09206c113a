"""GPU parity of the traversal loop with the transposition table on, redirects included
(omk_tt_select_redirect; reference src/mcts/mcts_engine_batch_tree_simple.cpp:88-165, the redirect
:142-156) against the CPU checker, which tests/test_oracle_redirect.py pins against a literal
restatement over node objects: paths, leaves, recorded moves, the node every child slot holds, virtual
loss, visit counts and the table's content bit for bit, search step after search step.  Games: the
reference's own collision fixture (tests/mcts/transposition_table_test.cpp:15-232, move lists [0, 1]
and [1, 0] share a key) and a stone-placing game whose key ignores the order of a side's stones."""
import numpy as np
import pytest

from oracle import ref_cpu as R
from tests.test_gpu_tt_policy import same_tables
from tests.test_oracle_redirect import fixture_tree, stones_tree

pytestmark = pytest.mark.gpu


def as_soa(g, rng, rave=False, mask_frac=0.0):
    n = g["n"]
    soa = dict(N=np.zeros(n, np.int32), W=np.zeros(n, np.float32), P=g["P"], VL=np.zeros(n, np.int32),
               child_begin=g["cb"], child_count=g["cc"], action=g["action"], hash=g["keys"])
    if rave:
        soa["rN"] = rng.integers(0, 30, n).astype(np.int32)
        soa["rW"] = (rng.uniform(-1, 1, n) * soa["rN"]).astype(np.float32)
    if mask_frac:
        bits = rng.random(n) >= mask_frac
        bits[0] = True
        pad = np.zeros((n + 31) // 32 * 32, np.uint8)
        pad[:n] = bits
        soa["legal"] = np.packbits(pad.reshape(-1, 32), axis=1, bitorder="little").view("<u4").reshape(-1).copy()
    return soa


def search_both(g, seed, batches, B, vl=3, max_depth=8, rave=False, mask_frac=0.0, log2=12, roots=None, revert_every=0):
    import omoknuni_small_amd as omk
    rng = np.random.default_rng(seed)
    soa = as_soa(g, rng, rave, mask_frac)
    n = g["n"]
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa)
    tt, ref_tt = omk.TranspositionTable(f, log2), R.RefTT(log2)
    alias = np.full(n, -1, np.int32)
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=vl, use_rave=rave, rave_k=300.0)
    rp = R.make_params(c_puct=1.4, virtual_loss=vl, use_rave=rave, rave_k=300.0, max_depth=max_depth)
    b = omk.Batch(f, B, max_depth)
    roots = np.zeros(B, np.int32) if roots is None else np.ascontiguousarray(roots, np.int32)
    total = np.zeros(5, np.int64)
    for step in range(batches):
        what = "seed %d step %d" % (seed, step)
        b.set_roots(roots)
        moves, counts = tt.select_redirect(b, sp)
        paths, plen, leaf, _ = b.read()
        rpaths, rplen, rleaf, rmoves, rcounts = ref.select_redirect_batch(roots, rp, ref_tt, g["keys"], alias)
        assert (plen == rplen).all(), what
        assert (paths == rpaths).all() and (leaf == rleaf).all(), what
        assert (moves == rmoves).all(), what
        assert counts == tuple(int(x) for x in rcounts), what
        total += rcounts
        assert (f.download_redirects() == alias).all(), what
        assert (f.download()["VL"] == ref.VL).all(), what
        same_tables(tt, ref_tt, what)
        if revert_every and step % revert_every == revert_every - 1:
            # a batch that is given up: the virtual losses come off again, nothing is backed up
            b.revert_vl(vl)
            ref.revert_vl_paths(rpaths, rplen, vl)
            assert (f.download()["VL"] == ref.VL).all(), what
            continue
        values = rng.uniform(-1, 1, B).astype(np.float32)
        b.set_values(values)
        b.backup(vl)
        ref.backup_batch(rpaths, rplen, values, vl)
        dev = f.download()
        assert (dev["N"] == ref.N).all() and (dev["VL"] == ref.VL).all(), what
        # the device adds a node's values of one step in another order than the serial loop
        assert np.allclose(dev["W"], ref.W, rtol=0, atol=1e-5 * max(1.0, np.sqrt(B))), what
        ref.W[:] = dev["W"]
    return f, ref, alias, total, (b, sp, tt)


@pytest.mark.parametrize("seed", [1, 2])
def test_collision_fixture_of_the_reference(seed):
    g = fixture_tree(np.random.default_rng(seed))
    f, ref, alias, total, _ = search_both(g, seed, batches=12, B=8)
    assert total[3] >= 1 and (alias >= 0).any()


@pytest.mark.parametrize("seed,vl,rave,mask", [(11, 3, False, 0.0), (12, 1, True, 0.0), (13, 0, False, 0.0),
                                               (14, 3, False, 0.25), (15, 2, True, 0.2)])
def test_stone_game_with_many_transpositions(seed, vl, rave, mask):
    g = stones_tree(np.random.default_rng(seed), cells=6, plies=4)
    f, ref, alias, total, _ = search_both(g, seed, batches=20, B=32, vl=vl, max_depth=6, rave=rave, mask_frac=mask)
    assert total[3] >= 5, total


def test_wide_nodes_and_a_depth_bound():
    # 70 children at the root and 69 under each: more than one round of 64 slots per node; paths cut at 2 steps
    g = stones_tree(np.random.default_rng(21), cells=70, plies=2)
    f, ref, alias, total, _ = search_both(g, 21, batches=6, B=96, max_depth=2, log2=14)
    assert total[4] == 6 * 96 * 2
    g = stones_tree(np.random.default_rng(22), cells=6, plies=4)
    search_both(g, 22, batches=8, B=16, max_depth=2)


def test_wide_nodes_with_transpositions():
    # the same wide tree with the positions [a, b] and [b, a] given one key: slots of nodes of more than 64
    # slots get re-pointed, and later selections read through them (the walk's path for wide nodes)
    g = stones_tree(np.random.default_rng(23), cells=70, plies=2)
    at = {tuple(h): i for i, h in enumerate(g["hist"])}
    for (x, y), i in [(k, v) for k, v in at.items() if len(k) == 2]:
        if x > y:
            g["keys"][i] = g["keys"][at[(y, x)]]
    f, ref, alias, total, _ = search_both(g, 23, batches=14, B=128, max_depth=2, log2=14)
    assert total[3] >= 10, total
    assert (alias >= 0).sum() >= 10


def test_a_transposition_to_an_ancestor_makes_paths_that_loop_up_to_the_depth_bound():
    # the position three plies down carries the key of the position one ply down (a repetition): once the
    # latter has visits the former's slot is re-pointed at it, and a path that comes that way goes round
    # until the depth bound ends it; a node then occurs several times on one path, and the backup counts
    # every occurrence, as the reference's loop over the path does
    g = fixture_tree(np.random.default_rng(51))
    for a, b in (([0, 0, 0], [0]), ([1, 1, 0], [1]), ([0, 1, 1], [0])):
        g["keys"][g["hist"].index(a)] = g["keys"][g["hist"].index(b)]
    f, ref, alias, total, _ = search_both(g, 51, batches=14, B=8, max_depth=9)
    assert total[3] >= 1
    looped = [int(s) for s in np.nonzero(alias >= 0)[0] if len(g["hist"][alias[s]]) < len(g["hist"][s])]
    assert looped, alias
    assert total[4] > 14 * 8 * 4          # paths longer than the game is deep


def test_several_roots_positions_without_a_key_and_batches_given_up():
    rng = np.random.default_rng(61)
    g = stones_tree(rng, cells=6, plies=4)
    g["keys"][rng.random(g["n"]) < 0.15] = np.uint64(0xFFFFFFFFFFFFFFFF)      # positions the host never keyed
    # traversals that start at the root and at two of its children (searches of three positions side by side)
    roots = np.array([0, 1, 2] * 8, np.int32)
    f, ref, alias, total, _ = search_both(g, 61, batches=24, B=24, max_depth=5, roots=roots, revert_every=5)
    assert total[3] >= 3, total


def test_a_table_that_runs_full_is_reported_and_the_traversals_are_made_all_the_same():
    # 16 slots for a game with far more positions: entries that find no room are dropped (and counted), the
    # traversals go on without them; the call reports the table as full after it has done everything else,
    # so the batch can be read, backed up or given up as after any other selection
    import omoknuni_small_amd as omk
    rng = np.random.default_rng(71)
    g = stones_tree(rng, cells=6, plies=3)
    soa = as_soa(g, rng)
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa)
    tt, ref_tt = omk.TranspositionTable(f, 4), R.RefTT(4)
    alias = np.full(g["n"], -1, np.int32)
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=2)
    rp = R.make_params(c_puct=1.4, virtual_loss=2, max_depth=5)
    B = 24
    b = omk.Batch(f, B, 5)
    roots = np.zeros(B, np.int32)
    full = 0
    for step in range(6):
        what = "step %d" % step
        b.set_roots(roots)
        dev_full = ref_full = False
        try:
            tt.select_redirect(b, sp)
        except omk.OmkError as e:
            assert "table full" in str(e), e
            dev_full = True
        try:
            rpaths, rplen, rleaf, rmoves, rcounts = ref.select_redirect_batch(roots, rp, ref_tt, g["keys"], alias)
        except ValueError as e:
            ref_full = True
            rpaths, rplen, rleaf, rmoves, rcounts = e.result
        assert dev_full == ref_full, what
        full += dev_full
        paths, plen, leaf, _ = b.read()
        assert (plen == rplen).all() and (paths == rpaths).all() and (leaf == rleaf).all(), what
        assert (f.download_redirects() == alias).all(), what
        assert (f.download()["VL"] == ref.VL).all(), what
        same_tables(tt, ref_tt, what)
        if step % 2:
            b.revert_vl(2)
            ref.revert_vl_paths(rpaths, rplen, 2)
        else:
            values = rng.uniform(-1, 1, B).astype(np.float32)
            b.set_values(values)
            b.backup(2)
            ref.backup_batch(rpaths, rplen, values, 2)
            dev = f.download()
            assert (dev["N"] == ref.N).all(), what
            assert np.allclose(dev["W"], ref.W, rtol=0, atol=1e-5 * max(1.0, np.sqrt(B))), what
            ref.W[:] = dev["W"]
        assert (f.download()["VL"] == ref.VL).all(), what
    assert full >= 3, full


def test_a_redirected_forest_is_a_graph_until_the_next_upload():
    import omoknuni_small_amd as omk
    rng = np.random.default_rng(31)
    g = stones_tree(rng, cells=5, plies=4)
    f, ref, alias, total, (b, sp, tt) = search_both(g, 31, batches=25, B=16, max_depth=6)
    assert total[3] > 0
    # what needs a tree says so
    b.set_roots(np.zeros(16, np.int32))
    with pytest.raises(omk.OmkError, match="re-pointed"):
        b.select(sp)
    with pytest.raises(omk.OmkError, match="re-pointed"):
        f.compact(0)
    # the root's action probabilities count the visits of the nodes its slots hold
    held = np.where(alias >= 0, alias, np.arange(g["n"])).astype(np.int32)
    seen = R.RefTree(N=ref.N[held], W=ref.W, P=ref.P, VL=ref.VL, child_begin=g["cb"], child_count=g["cc"],
                     action=g["action"])
    for root in [0] + [int(i) for i in np.nonzero(alias >= 0)[0][:3] if g["cc"][i] > 0]:
        got, k = f.action_probabilities(root, 1.0, 5)
        want, rk = seen.action_probabilities(root, 1.0, 5)
        assert k == rk and got.tobytes() == want.tobytes()
    # an upload brings a tree back
    soa = as_soa(g, rng)
    f.upload(soa)
    assert (f.download_redirects() == -1).all()
    b.set_roots(np.zeros(16, np.int32))
    b.select(sp)
    paths, plen, leaf, _ = b.read()
    rpaths, rplen, rleaf, _ = R.RefTree.from_soa(soa).select_batch(np.zeros(16, np.int32), R.make_params(max_depth=6))
    assert (paths == rpaths).all() and (plen == rplen).all()


def test_without_position_keys_or_with_widening_it_refuses():
    import omoknuni_small_amd as omk
    g = fixture_tree(np.random.default_rng(41))
    soa = as_soa(g, np.random.default_rng(41))
    del soa["hash"]
    f = omk.Forest.from_soa(soa)
    tt = omk.TranspositionTable(f, 8)
    b = omk.Batch(f, 4, 4)
    b.set_roots(np.zeros(4, np.int32))
    with pytest.raises(omk.OmkError, match="position keys"):
        tt.select_redirect(b, omk.SelectParams())
    f2 = omk.Forest.from_soa(as_soa(g, np.random.default_rng(41)))
    tt2 = omk.TranspositionTable(f2, 8)
    b2 = omk.Batch(f2, 4, 4)
    b2.set_roots(np.zeros(4, np.int32))
    with pytest.raises(omk.OmkError, match="widening"):
        tt2.select_redirect(b2, omk.SelectParams(pw=True))
