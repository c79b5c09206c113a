"""Randomised parity over whole sessions, the way an engine uses the library, against the CPU checker:
(1) one forest with two batches alive: roots set again (one root, sorted, unsorted; one to twelve thousand
traversals), selects interleaved between the batches, backups and reverts, statistics put back by an upload of
the same structure, batches destroyed and created again, statistics and timeline switched on and off;
(2) a tree that grows from its root: select, expansion with progressive widening and policies of every length
setPriorProbabilities distinguishes, backup, move probabilities, and tree reuse (re-root at the most visited
child, compaction, allocating or static) every few steps, under depth bounds short enough to be hit.
Paths, leaves, moves, new node ids, N and VL are exact; W within the bound of the full-size tests."""
import numpy as np
import pytest

from oracle import ref_cpu as R
from tests.helpers import random_tree
from tests.test_gpu_expand import offers
from tests.test_gpu_scheduler import layered_forest

pytestmark = pytest.mark.gpu


def same_statistics(f, ref, what, k):
    st = f.download()
    assert (st["N"] == ref.N).all() and (st["VL"] == ref.VL).all(), what
    err = np.abs(st["W"].astype(np.float64) - ref.W) / np.maximum(np.abs(ref.W), 1.0)
    assert err.max() <= 1e-5 * max(1.0, np.sqrt(k)), (what, err.max())   # k values summed per node in another order
    ref.W[:] = st["W"]


def two_batches_session(seed):
    import omoknuni_small_amd as omk
    rng = np.random.default_rng(seed)
    rave = bool(rng.integers(2))
    if rng.random() < 0.5:
        lay = [int(rng.integers(4, 300)), int(rng.integers(4, 30)), int(rng.integers(2, 6))]
        soa, roots = layered_forest(int(rng.integers(1 << 30)), lay, n_trees=int(rng.integers(1, 6)), rave=rave)
        D = 4
    else:
        soa, roots = random_tree(int(rng.integers(1 << 30)), n_expand=int(rng.integers(20, 300)),
                                 fanout=(1, int(rng.integers(2, 90))), max_depth=int(rng.integers(3, 9)), rave=rave,
                                 mask_frac=float(rng.choice([0, 0.3])), vl_frac=0.1, tie_frac=0.1,
                                 n_max=int(rng.integers(2, 400)))
        roots = np.asarray(roots, np.int32)
        D = 10
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa)
    caps = [int(rng.integers(64, 12000)), int(rng.integers(64, 12000))]
    bs = [omk.Batch(f, caps[0], D), omk.Batch(f, caps[1], D)]
    vl = int(rng.integers(1, 5))
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=vl, use_rave=rave, rave_k=500.0)
    rp = R.make_params(c_puct=1.4, virtual_loss=vl, use_rave=rave, rave_k=500.0, max_depth=D)
    cur = [None, None]
    for op in range(int(rng.integers(6, 16))):
        i = int(rng.integers(2))
        b = bs[i]
        what = "seed %d operation %d" % (seed, op)
        if cur[i] is None or rng.random() < 0.4:
            B = int(rng.integers(1, caps[i] + 1))
            mode = int(rng.integers(3))
            if mode == 0:
                tr = np.full(B, roots[int(rng.integers(len(roots)))], np.int32)
            elif mode == 1:
                tr = np.sort(rng.choice(roots, B)).astype(np.int32)
            else:
                tr = rng.choice(roots, B).astype(np.int32)
            b.set_roots(tr)
            cur[i] = tr
        if rng.random() < 0.3:
            b.enable_stats(bool(rng.integers(2)))
        if rng.random() < 0.2:
            b.enable_trace(bool(rng.integers(2)))
        tr = cur[i]
        rpaths, rlen, rleaf, _ = ref.select_batch(tr, rp, near_ties=False)
        b.select(sp)
        gpaths, glen, gleaf, _ = b.read()
        assert (gpaths == rpaths).all() and (glen == rlen).all() and (gleaf == rleaf).all(), what
        assert (f.download()["VL"] == ref.VL).all(), what
        if rng.random() < 0.25:
            b.revert_vl(vl)
            ref.revert_vl_paths(rpaths, rlen, vl)
        else:
            vals = rng.uniform(-1, 1, len(tr)).astype(np.float32)
            b.set_values(vals)
            b.backup(vl)
            ref.backup_batch(rpaths, rlen, vals, vl)
        same_statistics(f, ref, what, len(tr))
        if rng.random() < 0.15:      # the statistics put back: same structure, the batches stay usable
            soa2 = dict(soa)
            soa2["N"], soa2["W"], soa2["VL"] = ref.N.copy(), ref.W.copy(), ref.VL.copy()
            f.upload(soa2)
        if rng.random() < 0.15:      # a batch goes, another one comes (and may get the memory the old one had)
            j = int(rng.integers(2))
            bs[j].close()
            caps[j] = int(rng.integers(64, 12000))
            bs[j] = omk.Batch(f, caps[j], D)
            cur[j] = None
    for b in bs:
        b.close()
    f.close()


def growing_tree_session(seed):
    import omoknuni_small_amd as omk
    rng = np.random.default_rng(seed)
    A = int(rng.integers(9, 200))
    B = int(rng.integers(1, 5000)) if rng.random() < 0.6 else int(rng.integers(1, 100))
    D = int(rng.integers(4, 16))
    vl = int(rng.integers(1, 5))
    widening = (2.0, 0.5) if rng.random() < 0.5 else None
    soa = dict(N=np.zeros(1, np.int32), W=np.zeros(1, np.float32), P=np.ones(1, np.float32), VL=np.zeros(1, np.int32),
               child_begin=np.zeros(1, np.int32), child_count=np.zeros(1, np.int32), action=np.full(1, -1, np.int32))
    ref = R.RefTree.from_soa(soa)
    f = omk.Forest.from_soa(soa, capacity=2_000_000)
    b = omk.Batch(f, B, D)
    roots = np.zeros(B, np.int32)
    b.set_roots(roots)
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=vl)
    rp = R.make_params(c_puct=1.4, virtual_loss=vl, max_depth=D)
    max_moves = int(rng.integers(2, min(A, 60) + 1))
    for step in range(int(rng.integers(6, 16))):
        what = "seed %d step %d" % (seed, step)
        rpaths, rlen, rleaf, _ = ref.select_batch(roots, rp, near_ties=False)
        b.select(sp)
        gpaths, glen, gleaf, gact = b.read()
        assert (gpaths == rpaths).all() and (glen == rlen).all() and (gleaf == rleaf).all(), what
        assert (gact == ref.gather_actions(rpaths, rlen)).all(), what
        begin, moves, policy = offers(rng, rleaf, A, max_moves=max_moves)
        pb, pol = [0], []
        for t in range(B):
            k = begin[t + 1] - begin[t]
            mode = int(rng.integers(4))
            row = (policy[t] if mode == 0 else rng.random(k).astype(np.float32) if mode == 1
                   else rng.random(3).astype(np.float32) if mode == 2 else np.zeros(0, np.float32))
            pol.extend(row.tolist())
            pb.append(len(pol))
        pol, pb = np.array(pol if pol else [0.0], np.float32), np.array(pb, np.int32)
        rfirst = ref.expand_batch(rleaf, begin, moves, policy=pol, action_space=A, policy_begin=pb, widening=widening)
        gfirst = b.expand_ex(begin, moves, policy_begin=pb, policy=pol, action_space=A, widening=widening)
        assert (gfirst == rfirst).all(), what
        values = rng.uniform(-1, 1, B).astype(np.float32)
        ref.backup_batch(rpaths, rlen, values, vl)
        b.set_values(values)
        b.backup(vl)
        sx = f.download_structure()
        assert f.node_count()[0] == ref.n, what
        assert (sx["child_begin"] == ref.child_begin).all() and (sx["child_count"] == ref.child_count).all(), what
        assert (sx["action"] == ref.action).all() and f.download()["P"].tobytes() == ref.P.tobytes(), what
        same_statistics(f, ref, what, B)
        for temp in (0.001, 1.0):
            want, wn = ref.action_probabilities(0, temp, A)
            got, gn = f.action_probabilities(0, temp, A)
            assert gn == wn and got.tobytes() == want.tobytes(), what
        if ref.child_count[0] > 0 and rng.random() < 0.25:
            kids = np.arange(ref.child_begin[0], ref.child_begin[0] + ref.child_count[0])
            move = int(ref.action[kids[np.argmax(ref.N[kids])]])
            rc, gc = ref.reroot_child(0, move), f.reroot_child(0, move)
            assert rc == gc >= 0, what
            ref, order = ref.compacted(rc)
            gorder = f.compact(gc, static=bool(rng.integers(2)) and f.node_count()[0] <= 1_000_000)
            assert (gorder == order).all() and f.node_count()[0] == ref.n, what
            b.set_roots(roots)
    b.close()
    f.close()


@pytest.mark.parametrize("first", [0, 20])
def test_two_batches_on_one_forest(first):
    for seed in range(first, first + 20):
        two_batches_session(seed)


@pytest.mark.parametrize("first", [0, 15])
def test_a_tree_that_grows_and_is_reused(first):
    for seed in range(first, first + 15):
        growing_tree_session(seed)


def test_selections_that_give_up_in_mid_session():
    """Tiny spin limits make waiting wavefronts give up (the kernels still end normally): the library says so,
    and once the statistics are put back the same batch selects correctly again, time after time."""
    import omoknuni_small_amd as omk
    gave_up = 0
    for seed in range(12):
        rng = np.random.default_rng(seed)
        lay = [int(rng.integers(4, 300)), int(rng.integers(4, 30)), int(rng.integers(2, 8))]
        rave = bool(rng.integers(2))
        soa, roots = layered_forest(int(rng.integers(1 << 30)), lay, n_trees=int(rng.integers(1, 4)), rave=rave)
        B, D, vl = int(rng.integers(200, 12000)), 4, 3
        troots = roots[np.sort(rng.integers(0, len(roots), B))].astype(np.int32)
        ref = R.RefTree.from_soa(soa)
        f = omk.Forest.from_soa(soa)
        b = omk.Batch(f, B, D)
        b.set_roots(troots)
        sp = omk.SelectParams(c_puct=1.4, virtual_loss=vl, use_rave=rave, rave_k=1000.0)
        rp = R.make_params(c_puct=1.4, virtual_loss=vl, use_rave=rave, rave_k=1000.0, max_depth=D)
        for op in range(5):
            if rng.random() < 0.5:
                cur = dict(soa)
                cur["N"], cur["W"], cur["VL"] = ref.N.copy(), ref.W.copy(), ref.VL.copy()
                b.set_spin_limit(int(rng.choice([0, 1, 2, 5, 20, 100])))
                b.select(sp)
                try:
                    b.read()
                except omk.OmkError as e:
                    assert e.code == -6, e       # OMK_ERR_STATE: the selection gave up
                    gave_up += 1
                f.upload(cur)                    # whatever virtual loss the incomplete selection left is gone
                b.set_spin_limit(1 << 22)
            rpaths, rlen, rleaf, _ = ref.select_batch(troots, rp, near_ties=False)
            b.select(sp)
            gpaths, glen, gleaf, _ = b.read()
            assert (gpaths == rpaths).all() and (glen == rlen).all() and (gleaf == rleaf).all(), (seed, op)
            vals = rng.uniform(-1, 1, B).astype(np.float32)
            ref.backup_batch(rpaths, rlen, vals, vl)
            b.set_values(vals)
            b.backup(vl)
            same_statistics(f, ref, "seed %d operation %d" % (seed, op), B)
        b.close()
        f.close()
    assert gave_up >= 5
