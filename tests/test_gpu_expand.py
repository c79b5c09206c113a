"""GPU parity of leaf expansion (omk_expand_batch) and of search steps on a tree that grows on
the device: select -> leaf gather -> expand -> backup, every array against the CPU checker
after every phase.  Structure, priors, actions, N and virtual loss bit-exact; W within 1e-5 (relative to
max(|W|, 1); where hundreds of values meet at a node in one step, the bound grows with the square root of
their number, as in the full-size tests: the device adds them in another order than the serial loop)."""
import numpy as np
import pytest

from oracle import ref_cpu as R
from tests.helpers import random_tree

pytestmark = pytest.mark.gpu


def assert_same_forest(f, ref, what, k=1):
    """k: values a node may have taken in the step just backed up (the device adds them in another order than
    the serial loop; the bound grows with sqrt(k), as in the full-size tests)."""
    st = f.download()
    sx = f.download_structure()
    assert len(st["N"]) == ref.n, what
    assert (sx["child_begin"] == ref.child_begin).all() and (sx["child_count"] == ref.child_count).all(), what
    assert (sx["action"] == ref.action).all(), what
    assert st["P"].tobytes() == ref.P.tobytes(), what
    assert (st["N"] == ref.N).all() and (st["VL"] == ref.VL).all(), what
    err = np.abs(st["W"].astype(np.float64) - ref.W) / np.maximum(np.abs(ref.W), 1.0)
    assert err.max() <= 1e-5 * max(1.0, np.sqrt(k) / 8.0), what
    return st


def offers(rng, leaves, action_space, terminal_frac=0.1, max_moves=40):
    """Legal moves per traversal, a function of the leaf so that two traversals at one leaf
    offer the same state's moves, plus a policy row per traversal."""
    begin, moves = [0], []
    for lf in leaves:
        r = np.random.default_rng(int(lf) * 7919 + 13)
        if r.random() < terminal_frac:
            k = 0
        else:
            k = int(r.integers(1, max_moves + 1))
        moves.extend(r.choice(action_space, size=k, replace=False).tolist())
        begin.append(len(moves))
    policy = rng.random((len(leaves), action_space)).astype(np.float32)
    policy /= policy.sum(axis=1, keepdims=True)
    return np.array(begin, np.int32), np.array(moves, np.int32), policy


@pytest.mark.parametrize("rave,B", [(False, 96), (True, 700)])
def test_tree_grows_on_the_device(rave, B):
    import omoknuni_small_amd as omk
    A = 81
    soa = dict(N=np.zeros(1, np.int32), W=np.zeros(1, np.float32), P=np.ones(1, np.float32), VL=np.zeros(1, np.int32),
               child_begin=np.zeros(1, np.int32), child_count=np.zeros(1, np.int32), action=np.full(1, -1, np.int32))
    if rave:
        soa["rN"] = np.zeros(1, np.int32)
        soa["rW"] = np.zeros(1, np.float32)
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa, capacity=400_000)
    D, vl = 12, 3
    b = omk.Batch(f, B, D)
    roots = np.zeros(B, np.int32)
    b.set_roots(roots)
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=vl, use_rave=rave, rave_k=1000.0)
    rp = R.make_params(c_puct=1.4, virtual_loss=vl, use_rave=rave, rave_k=1000.0, max_depth=D)
    rng = np.random.default_rng(4)
    for step in range(14):
        rpaths, rlen, rleaf, near = ref.select_batch(roots, rp)
        b.select(sp)
        gpaths, glen, gleaf, gact = b.read()
        bad = np.nonzero((gpaths != rpaths).any(axis=1) | (glen != rlen) | (gleaf != rleaf))[0]
        assert len(bad) == 0, "step %d: %d paths differ (near ties flagged %d)" % (step, len(bad), int((near >= 0).sum()))
        begin, moves, policy = offers(rng, rleaf, A)
        pol = policy if step % 3 else None          # every third step: no policy, uniform priors
        rfirst = ref.expand_batch(rleaf, begin, moves, policy=pol, action_space=A)
        gfirst = b.expand(begin, moves, policy=pol, action_space=A)
        assert (gfirst == rfirst).all(), "step %d: new ids differ" % step
        assert_same_forest(f, ref, "after expansion, step %d" % step)
        values = rng.uniform(-1, 1, B).astype(np.float32)
        ref.backup_batch(rpaths, rlen, values, vl)
        b.set_values(values)
        b.backup(vl)
        st = assert_same_forest(f, ref, "after backup, step %d" % step, B)
        ref.W[:] = st["W"]
    assert ref.n > 1000


def test_leaves_at_the_depth_bound_are_left_alone_and_take_no_ids():
    """With a short depth bound the selection soon stops at nodes that have children already; the host still
    offers their states' moves.  Such a node stays as it is and no ids are spent on it: the ids of the nodes
    that ARE created stay those of the checker, step after step."""
    import omoknuni_small_amd as omk
    A, B, D, vl = 64, 600, 3, 3
    soa = dict(N=np.zeros(1, np.int32), W=np.zeros(1, np.float32), P=np.ones(1, np.float32), VL=np.zeros(1, np.int32),
               child_begin=np.zeros(1, np.int32), child_count=np.zeros(1, np.int32), action=np.full(1, -1, np.int32))
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa, capacity=400_000)
    b = omk.Batch(f, B, D)
    roots = np.zeros(B, np.int32)
    b.set_roots(roots)
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=vl)
    rp = R.make_params(c_puct=1.4, virtual_loss=vl, max_depth=D)
    rng = np.random.default_rng(8)
    capped = 0
    for step in range(12):
        rpaths, rlen, rleaf, _ = ref.select_batch(roots, rp)
        b.select(sp)
        gpaths, glen, gleaf, _ = b.read()
        assert (gpaths == rpaths).all() and (gleaf == rleaf).all()
        capped += int((ref.child_count[rleaf] > 0).sum())
        begin, moves, policy = offers(rng, rleaf, A, max_moves=20)
        rfirst = ref.expand_batch(rleaf, begin, moves, policy=policy, action_space=A)
        gfirst = b.expand(begin, moves, policy=policy, action_space=A)
        assert (gfirst == rfirst).all(), "step %d: new ids differ" % step
        assert f.node_count()[0] == ref.n
        values = rng.uniform(-1, 1, B).astype(np.float32)
        ref.backup_batch(rpaths, rlen, values, vl)
        b.set_values(values)
        b.backup(vl)
        st, sx = f.download(), f.download_structure()
        assert (sx["child_begin"] == ref.child_begin).all() and (sx["child_count"] == ref.child_count).all()
        assert (st["N"] == ref.N).all() and (st["VL"] == ref.VL).all() and st["P"].tobytes() == ref.P.tobytes()
        # (600 values a step meet at the root, added in another order than the serial loop's)
        err = np.abs(st["W"].astype(np.float64) - ref.W) / np.maximum(np.abs(ref.W), 1.0)
        assert err.max() <= 1e-5 * np.sqrt(B), step
        ref.W[:] = st["W"]
    assert capped > 100          # the bound was hit at nodes that have children


def test_tree_grows_with_progressive_widening_and_ragged_policies():
    """The reference's default settings (use_progressive_widening, c = 2, k = 0.5): only the first
    min(legal, max(8, 2 sqrt(N + 1))) offered moves become children; policies of every length
    setPriorProbabilities distinguishes (action space, number of children, neither, empty)."""
    import omoknuni_small_amd as omk
    A, B, D, vl = 120, 400, 10, 3
    soa = dict(N=np.zeros(1, np.int32), W=np.zeros(1, np.float32), P=np.ones(1, np.float32), VL=np.zeros(1, np.int32),
               child_begin=np.zeros(1, np.int32), child_count=np.zeros(1, np.int32), action=np.full(1, -1, np.int32))
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa, capacity=300_000)
    b = omk.Batch(f, B, D)
    roots = np.zeros(B, np.int32)
    b.set_roots(roots)
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=vl)
    rp = R.make_params(c_puct=1.4, virtual_loss=vl, max_depth=D)
    rng = np.random.default_rng(8)
    kinds_seen = set()
    for step in range(10):
        rpaths, rlen, rleaf, near = ref.select_batch(roots, rp)
        b.select(sp)
        gpaths, glen, gleaf, _ = b.read()
        assert (gpaths == rpaths).all() and (gleaf == rleaf).all(), "step %d" % step
        begin, moves, _ = offers(rng, rleaf, A, max_moves=60)
        # a policy per traversal, its length a function of the leaf (two traversals at one leaf agree)
        pb, pol = [0], []
        for t, lf in enumerate(rleaf):
            legal = int(begin[t + 1] - begin[t])
            made = R.lib().ref_widened_children(min(legal, 1000), int(ref.N[lf]), 1, 2.0, 0.5) if legal else 0
            kind = int(lf) % 4
            size = [A, made, made + 3, 0][kind]
            kinds_seen.add(kind)
            pol.extend(np.random.default_rng(int(lf) + 5).uniform(-0.2, 1.2, size).astype(np.float32).tolist())
            pb.append(len(pol))
        pol = np.array(pol, np.float32)
        rfirst = ref.expand_batch(rleaf, begin, moves, policy=pol, action_space=A, policy_begin=pb, widening=(2.0, 0.5))
        gfirst = b.expand_ex(begin, moves, policy_begin=pb, policy=pol, action_space=A, widening=(2.0, 0.5))
        assert (gfirst == rfirst).all(), "step %d: new ids differ" % step
        assert_same_forest(f, ref, "after expansion, step %d" % step)
        values = rng.uniform(-1, 1, B).astype(np.float32)
        ref.backup_batch(rpaths, rlen, values, vl)
        b.set_values(values)
        b.backup(vl)
        st = assert_same_forest(f, ref, "after backup, step %d" % step, B)
        ref.W[:] = st["W"]
    assert kinds_seen == {0, 1, 2, 3} and ref.n > 500
    # widening at work: no node has more children than its visit count allowed when it was expanded
    cc = ref.child_count[ref.child_count > 0]
    assert cc.max() <= 60 and (cc >= 1).all() and (cc[cc < 8] >= 1).all()


def test_expand_on_an_uploaded_tree_with_mask_and_shared_leaves():
    import omoknuni_small_amd as omk
    soa, roots = random_tree(77, n_expand=60, fanout=(2, 9), max_depth=5, mask_frac=0.2)
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa, capacity=len(soa["N"]) + 5000)
    B, D = 300, 8
    b = omk.Batch(f, B, D)
    troots = np.full(B, roots[0], np.int32)
    b.set_roots(troots)
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=3)
    rp = R.make_params(c_puct=1.4, virtual_loss=3, max_depth=D)
    rpaths, rlen, rleaf, _ = ref.select_batch(troots, rp)
    b.select(sp)
    _, _, gleaf, _ = b.read()
    assert (gleaf == rleaf).all()
    assert len(np.unique(rleaf)) < B            # several traversals share a leaf
    begin, moves, policy = offers(np.random.default_rng(1), rleaf, 50)
    policy[:, 7] = 1.5                          # clamped to 1
    policy[:, 8] = -0.5                         # clamped to 0
    moves[::11] = 60                            # outside the action space: default prior
    rfirst = ref.expand_batch(rleaf, begin, moves, policy=policy, action_space=50)
    gfirst = b.expand(begin, moves, policy=policy, action_space=50)
    assert (gfirst == rfirst).all()
    assert_same_forest(f, ref, "after expansion")
    assert (f.download_structure()["child_count"] == ref.child_count).all()
    # the mask now covers the new nodes: select again and compare
    values = np.zeros(B, np.float32)
    ref.backup_batch(rpaths, rlen, values, 3)
    b.set_values(values)
    b.backup(3)
    rpaths, rlen, rleaf, _ = ref.select_batch(troots, rp)
    b.select(sp)
    gpaths, glen, gleaf, _ = b.read()
    assert (gpaths == rpaths).all() and (gleaf == rleaf).all()


def test_expand_beyond_capacity_changes_nothing():
    import omoknuni_small_amd as omk
    soa = dict(N=np.zeros(1, np.int32), W=np.zeros(1, np.float32), P=np.ones(1, np.float32), VL=np.zeros(1, np.int32),
               child_begin=np.zeros(1, np.int32), child_count=np.zeros(1, np.int32), action=np.full(1, -1, np.int32))
    f = omk.Forest.from_soa(soa, capacity=4)
    b = omk.Batch(f, 2, 4)
    b.set_roots(np.zeros(2, np.int32))
    b.select(omk.SelectParams())
    b.read()
    with pytest.raises(omk.OmkError) as e:
        b.expand([0, 5, 5], [0, 1, 2, 3, 4])
    assert e.value.code == -3                    # OMK_ERR_CAPACITY
    assert f.node_count() == (1, 4)
    assert f.download_structure()["child_count"].tolist() == [0]
    first = b.expand([0, 3, 3], [0, 1, 2])
    assert first.tolist() == [1, -1] and f.node_count()[0] == 4


@pytest.mark.parametrize("mask_frac", [0.0, 0.3])
def test_action_probabilities_match_the_checker(mask_frac):
    """MCTSEngine::getActionProbabilities through the C ABI: bit-exact (the arithmetic runs on
    the host in the reference's order; the counts come from the device)."""
    import omoknuni_small_amd as omk
    soa, roots = random_tree(31, n_expand=50, fanout=(3, 30), max_depth=4, mask_frac=mask_frac, n_max=500)
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa)
    A = 40
    nodes = [int(roots[0])] + [int(i) for i in np.nonzero(soa["child_count"] > 0)[0][:10]] + \
            [int(np.nonzero(soa["child_count"] == 0)[0][0])]
    for node in nodes:
        for temp in (0.001, 0.5, 1.0, 2.0):
            rp, rn = ref.action_probabilities(node, temp, A)
            gp, gn = f.action_probabilities(node, temp, A)
            assert gn == rn and gp.tobytes() == rp.tobytes(), (node, temp)


@pytest.mark.parametrize("mask_frac,rave", [(0.0, False), (0.25, True)])
def test_reroot_and_compaction_match_the_checker(mask_frac, rave):
    """Tree reuse between moves: the child reached by the move becomes the root, the rest is
    dropped, the subtree is renumbered; searching goes on and still matches."""
    import omoknuni_small_amd as omk
    soa, roots = random_tree(41, n_expand=150, fanout=(2, 12), max_depth=6, mask_frac=mask_frac, rave=rave, n_max=300)
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa)
    root = int(roots[0])
    # the move: the action of the most visited child of the root
    kids = np.arange(soa["child_begin"][root], soa["child_begin"][root] + soa["child_count"][root])
    if "legal" in soa:
        kids = kids[((soa["legal"][kids >> 5] >> (kids & 31).astype(np.uint32)) & 1) == 1]
    move = int(soa["action"][kids[np.argmax(soa["N"][kids])]])
    rc, gc = ref.reroot_child(root, move), f.reroot_child(root, move)
    assert gc == rc >= 0
    assert f.reroot_child(root, 10_000) == ref.reroot_child(root, 10_000) == -1
    ref2, order = ref.compacted(rc)
    gorder = f.compact(gc)
    assert (gorder == order).all() and f.node_count()[0] == ref2.n
    assert_same_forest(f, ref2, "after compaction")
    # search on from the new root
    B, D = 200, 8
    b = omk.Batch(f, B, D)
    b.set_roots(np.zeros(B, np.int32))
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=3, use_rave=rave, rave_k=1000.0)
    rp = R.make_params(c_puct=1.4, virtual_loss=3, use_rave=rave, rave_k=1000.0, max_depth=D)
    rpaths, rlen, rleaf, _ = ref2.select_batch(np.zeros(B, np.int32), rp)
    b.select(sp)
    gpaths, glen, gleaf, _ = b.read()
    assert (gpaths == rpaths).all() and (gleaf == rleaf).all()
    assert (f.download()["VL"] == ref2.VL).all()


def test_rave_backup_matches_the_checker():
    """The RAVE part of MCTSEngine::backPropagate (not run by the reference's live loop; offered
    for engines that do): rN exact, rW within 1e-5."""
    import omoknuni_small_amd as omk
    soa, roots = random_tree(52, n_expand=120, fanout=(3, 14), max_depth=6, mask_frac=0.15, rave=True, n_max=200)
    # small action space, so that sibling subtrees share actions (what RAVE is about)
    soa["action"] = np.where(soa["action"] >= 0, soa["action"] % 9, soa["action"]).astype(np.int32)
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa)
    B, D = 500, 7
    b = omk.Batch(f, B, D)
    troots = np.full(B, roots[0], np.int32)
    b.set_roots(troots)
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=3, use_rave=True, rave_k=50.0)
    rp = R.make_params(c_puct=1.4, virtual_loss=3, use_rave=True, rave_k=50.0, max_depth=D)
    rng = np.random.default_rng(2)
    for step in range(3):
        rpaths, rlen, rleaf, _ = ref.select_batch(troots, rp)
        b.select(sp)
        gpaths, glen, gleaf, _ = b.read()
        assert (gpaths == rpaths).all(), "step %d" % step
        values = rng.uniform(-1, 1, B).astype(np.float32)
        b.set_values(values)
        ref.rave_backup_batch(rpaths, rlen, values)
        b.backup_rave()
        ref.backup_batch(rpaths, rlen, values, 3)
        b.backup(3)
        st = f.download()
        assert (st["rN"] == ref.rN).all() and ref.rN.sum() > soa["rN"].sum()
        err = np.abs(st["rW"].astype(np.float64) - ref.rW) / np.maximum(np.abs(ref.rW), 1.0)
        assert err.max() <= 1e-5
        assert (st["N"] == ref.N).all() and (st["VL"] == ref.VL).all()
        ref.W[:] = st["W"]
        ref.rW[:] = st["rW"]


def test_root_noise_matches_the_checker():
    import omoknuni_small_amd as omk
    soa, roots = random_tree(61, n_expand=40, fanout=(5, 60), max_depth=3, mask_frac=0.25)
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa)
    rng = np.random.default_rng(4)
    for node in (int(roots[0]), int(np.nonzero(soa["child_count"] > 0)[0][-1])):
        cb, cc = int(soa["child_begin"][node]), int(soa["child_count"][node])
        ids = np.arange(cb, cb + cc)
        n_children = int(((soa["legal"][ids >> 5] >> (ids & 31).astype(np.uint32)) & 1).sum())
        gamma = rng.gamma(0.3, 1.0, n_children).astype(np.float32)
        assert ref.add_root_noise(node, gamma, 0.25) == n_children
        f.add_root_noise(node, gamma, 0.25)
        assert (f.download()["P"] == ref.P).all()  # same operations in the same order: bit-exact
    with pytest.raises(omk.OmkError):
        f.add_root_noise(int(roots[0]), np.ones(1, np.float32), 0.25)


def test_compaction_of_deep_and_wide_shapes_and_of_a_broken_structure():
    """The level-by-level renumbering on shapes that stress it: a path-like tree (one node per
    level for hundreds of levels), one very wide level, the whole tree from its root; and child
    ranges that loop back, which are refused."""
    import omoknuni_small_amd as omk
    # a spine 300 levels deep with a few leaves on the way, then a node with 900 children
    N, cb, cc = [1], [0], [0]
    spine = 0
    for d in range(300):
        fan = 3 if d % 7 == 0 else 1
        cb[spine], cc[spine] = len(N), fan
        first = len(N)
        for _ in range(fan):
            N.append(d + 1); cb.append(0); cc.append(0)
        spine = first + fan - 1
    cb[spine], cc[spine] = len(N), 900
    for i in range(900):
        N.append(i); cb.append(0); cc.append(0)
    n = len(N)
    soa = dict(N=np.array(N, np.int32), W=np.arange(n, dtype=np.float32), P=np.full(n, 0.5, np.float32),
               VL=np.zeros(n, np.int32), child_begin=np.array(cb, np.int32), child_count=np.array(cc, np.int32),
               action=np.arange(n, dtype=np.int32))
    ref = R.RefTree.from_soa(soa)
    for new_root in (0, int(cb[0]) + 2, spine):
        f = omk.Forest.from_soa(soa)
        ref2, order = ref.compacted(new_root)
        gorder = f.compact(new_root)
        assert len(gorder) == len(order) and (gorder == order).all(), new_root
        assert_same_forest(f, ref2, "subtree of %d" % new_root)
    # a child range that points back at the root: not a tree
    bad = dict(soa)
    bad["child_begin"] = soa["child_begin"].copy()
    bad["child_count"] = soa["child_count"].copy()
    bad["child_begin"][n - 1], bad["child_count"][n - 1] = 0, 2
    with pytest.raises(omk.OmkError):  # the upload already refuses it (a node with two parents)
        omk.Forest.from_soa(bad).compact(0)


def test_stale_batch_is_refused_after_compaction():
    """Roots and paths are node ids: after a compaction a batch made before it says so."""
    import omoknuni_small_amd as omk
    soa, roots = random_tree(73, n_expand=80, fanout=(2, 8), max_depth=6)
    f = omk.Forest.from_soa(soa)
    b = omk.Batch(f, 50, 6)
    b.set_roots(np.zeros(50, np.int32))
    sp = omk.SelectParams()
    b.select(sp)
    f.compact(int(soa["child_begin"][0]))
    for call in (lambda: b.select(sp), lambda: b.backup(3), lambda: b.read(), lambda: b.revert_vl(3)):
        with pytest.raises(omk.OmkError) as e:
            call()
        assert e.value.code == -6
    b.set_roots(np.zeros(50, np.int32))
    b.select(sp)
    b.read()
    # an upload of the same child ranges as the last upload (statistics put back) keeps a batch
    # usable; an upload of anything else does not
    st = dict(f.download(), **f.download_structure())
    f.upload(st)
    b.set_roots(np.zeros(50, np.int32))
    b.select(sp)
    f.upload(st)
    b.select(sp)
    b.read()
    f.upload(soa)
    with pytest.raises(omk.OmkError) as e:
        b.select(sp)
    assert e.value.code == -6
