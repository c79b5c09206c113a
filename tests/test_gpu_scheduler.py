"""GPU parity for the parts of the selection kernel that only crowded trees reach: nodes with
a thousand visitors or more, which several wavefronts settle together (slices of the winner
order, shared partition), several such nodes at once, fan-outs beyond the widest node that
is settled that way, children whose score hardly moves with virtual loss (long runs of one
winner), and the bounded wait of the persistent kernel."""
import numpy as np
import pytest

from oracle import ref_cpu as R

pytestmark = pytest.mark.gpu


def layered_forest(seed, fans, n_trees=1, rave=False, plateau=False):
    """n_trees complete trees, level l has fan-out fans[l]; benchmark-like statistics."""
    rng = np.random.default_rng(seed)
    N, W, P, cb, cc, act, rN, rW = ([] for _ in range(8))
    roots = []

    def stats(k, parent_sorted=False):
        n = np.minimum(rng.zipf(1.2, k), 10_000).astype(np.int64)
        n[rng.random(k) < 0.2] = 0
        w = rng.uniform(-1, 1, k) * n
        logits = rng.normal(0, 1.5, k)
        p = np.exp(logits - logits.max())
        p /= p.sum()
        return n, w, p

    for _ in range(n_trees):
        roots.append(len(N))
        N.append(200_000); W.append(0.0); P.append(0.0); cb.append(0); cc.append(0); act.append(-1)
        rN.append(0); rW.append(0.0)
        level = [roots[-1]]
        for f in fans:
            nxt = []
            for node in level:
                n, w, p = stats(f)
                cb[node] = len(N)
                cc[node] = f
                for i in range(f):
                    nxt.append(len(N))
                    N.append(int(n[i])); W.append(float(w[i])); P.append(float(p[i]))
                    cb.append(0); cc.append(0); act.append(i)
                    r = int(min(rng.zipf(1.3), 5000))
                    rN.append(r); rW.append(float(rng.uniform(-1, 1) * r))
                if plateau:
                    # a few heavily visited children with a high blended value and a tiny prior:
                    # their score hardly moves with virtual loss
                    for i in rng.choice(f, 3, replace=False):
                        c = cb[node] + int(i)
                        N[c] = 9000; W[c] = 0.93 * 9000; P[c] = 1e-4; rN[c] = 4000; rW[c] = 0.95 * 4000
                N[node] = max(N[node], 1 + int(sum(N[cb[node] + i] for i in range(f))))
            level = nxt
    soa = dict(N=np.array(N, np.int32), W=np.array(W, np.float32), P=np.array(P, np.float32),
               VL=np.zeros(len(N), np.int32), child_begin=np.array(cb, np.int32), child_count=np.array(cc, np.int32),
               action=np.array(act, np.int32))
    if rave:
        soa["rN"] = np.array(rN, np.int32)
        soa["rW"] = np.array(rW, np.float32)
    return soa, np.array(roots, np.int32)


def select_both(soa, troots, D, vl=3, rave=False, rave_k=1000.0, steps=2):
    import omoknuni_small_amd as omk
    ref = R.RefTree.from_soa(soa)
    rp = R.make_params(c_puct=1.4, virtual_loss=vl, use_rave=rave, rave_k=rave_k, max_depth=D)
    f = omk.Forest.from_soa(soa)
    b = omk.Batch(f, len(troots), D)
    b.set_roots(troots)
    b.enable_stats()
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=vl, use_rave=rave, rave_k=rave_k)
    rng = np.random.default_rng(1)
    stats = None
    for step in range(steps):
        rpaths, rlen, rleaf, near = ref.select_batch(troots, rp)
        b.select(sp)
        gpaths, glen, gleaf, _ = b.read()
        bad = np.nonzero((gpaths != rpaths).any(axis=1) | (glen != rlen) | (gleaf != rleaf))[0]
        assert len(bad) == 0, "step %d: %d paths differ, first traversal %d (near ties flagged: %d)" % (
            step, len(bad), bad[0], int((near >= 0).sum()))
        assert (f.download()["VL"] == ref.VL).all()
        step_stats = b.stats()
        stats = step_stats if stats is None else {k: stats[k] + v for k, v in step_stats.items()}  # over all steps
        values = rng.uniform(-1, 1, len(troots)).astype(np.float32)
        ref.backup_batch(rpaths, rlen, values, vl)
        b.set_values(values)
        b.backup(vl)
        st = f.download()
        assert (st["N"] == ref.N).all() and (st["VL"] == ref.VL).all()
        ref.W[:] = st["W"]
    return stats


@pytest.mark.parametrize("fan,rave,plateau", [(300, False, False), (300, True, False), (300, True, True),
                                              (48, False, False), (362, True, True)])
def test_heavy_nodes_are_sliced(fan, rave, plateau):
    soa, roots = layered_forest(7, [fan, 40], rave=rave, plateau=plateau)
    st = select_both(soa, np.zeros(20_000, np.int32), 3, rave=rave)
    assert st["sliced_nodes"] >= 1, st
    assert st["replayed_nodes"] == 0, st


def test_fanout_beyond_the_sliced_path():
    # the root is wider than the widest node that several wavefronts share: one wavefront
    # settles its 6000 visitors batch after batch (its children may still be sliced)
    soa, roots = layered_forest(8, [700, 20])
    st = select_both(soa, np.zeros(6000, np.int32), 3)
    assert st["replayed_nodes"] == 0, st


def test_several_heavy_roots_at_once():
    soa, roots = layered_forest(9, [120, 30], n_trees=5, rave=True, plateau=True)
    troots = roots[np.arange(5 * 2500) % 5]
    st = select_both(soa, troots, 3, rave=True)
    assert st["sliced_nodes"] >= 5, st


def test_tiny_virtual_loss_many_visitors():
    soa, roots = layered_forest(10, [200, 25])
    select_both(soa, np.zeros(9000, np.int32), 3, vl=1)


def test_bounded_wait_reports_and_recovers():
    """A spin limit of zero makes every waiting wavefront give up at once: the kernel still
    ends normally, the selection is reported as incomplete, and the batch works again."""
    import omoknuni_small_amd as omk
    soa, roots = layered_forest(11, [60, 30, 10])
    troots = np.zeros(3000, np.int32)
    f = omk.Forest.from_soa(soa)
    b = omk.Batch(f, len(troots), 4)
    b.set_roots(troots)
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=3)
    b.set_spin_limit(0)
    b.select(sp)
    with pytest.raises(omk.OmkError) as e:
        b.read()
    assert e.value.code == -6, e.value  # OMK_ERR_STATE
    b.set_spin_limit(1 << 22)
    f.upload(soa)
    ref = R.RefTree.from_soa(soa)
    rpaths, rlen, rleaf, _ = ref.select_batch(troots, R.make_params(c_puct=1.4, virtual_loss=3, max_depth=4))
    b.select(sp)
    gpaths, glen, gleaf, _ = b.read()
    assert (gpaths == rpaths).all() and (gleaf == rleaf).all()
    assert (f.download()["VL"] == ref.VL).all()


def test_no_virtual_loss_with_thousands_of_visitors():
    """Without virtual loss nothing changes between visitors: all of them follow the first one
    down the same path, thousands per node (shared partition, no slices)."""
    soa, roots = layered_forest(12, [90, 30, 8])
    st = select_both(soa, np.zeros(5000, np.int32), 5, vl=0)
    assert st["sliced_nodes"] == 0, st   # slices need virtual loss; the partition is still shared


def test_two_selections_in_a_row_accumulate_virtual_loss():
    """select, select again without a backup in between (virtual loss of the first is still on
    the tree), then revert both: counters return to where they started."""
    import omoknuni_small_amd as omk
    soa, roots = layered_forest(13, [70, 25], rave=True)
    ref = R.RefTree.from_soa(soa)
    rp = R.make_params(c_puct=1.4, virtual_loss=3, use_rave=True, rave_k=1000.0, max_depth=3)
    f = omk.Forest.from_soa(soa)
    B = 2500
    b1, b2 = omk.Batch(f, B, 3), omk.Batch(f, B, 3)
    troots = np.zeros(B, np.int32)
    b1.set_roots(troots)
    b2.set_roots(troots)
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=3, use_rave=True, rave_k=1000.0)
    r1 = ref.select_batch(troots, rp)
    b1.select(sp)
    r2 = ref.select_batch(troots, rp)
    b2.select(sp)
    g1, g2 = b1.read(), b2.read()
    assert (g1[0] == r1[0]).all() and (g2[0] == r2[0]).all()
    assert (f.download()["VL"] == ref.VL).all() and ref.VL.max() > 0
    b2.revert_vl(3)
    b1.revert_vl(3)
    assert (f.download()["VL"] == 0).all()


def chain_forest(seed, depth, fan, dominate):
    """A spine of `depth` nodes: every spine node has `fan` children, one of which (the next
    spine node) carries most of the prior when `dominate`; the other children are leaves or
    have one level of children of their own."""
    rng = np.random.default_rng(seed)
    N, W, P, cb, cc, act = [1000], [0.0], [0.0], [0], [0], [-1]
    spine = 0
    for d in range(depth):
        first = len(N)
        cb[spine], cc[spine] = first, fan
        nxt = int(rng.integers(fan))
        pr = rng.dirichlet(np.ones(fan)).astype(np.float32)
        if dominate:
            pr = (pr * 0.05).astype(np.float32)
            pr[nxt] = np.float32(0.95)
        for i in range(fan):
            n = int(rng.integers(0, 30))
            N.append(n); W.append(float(np.float32(rng.uniform(-n, n)))); P.append(float(pr[i]))
            cb.append(0); cc.append(0); act.append(i)
        # some siblings get children too, so that visitors pushed off the spine walk on
        for i in range(fan):
            if i != nxt and rng.random() < 0.3:
                c = first + i
                cb[c], cc[c] = len(N), 3
                for j in range(3):
                    N.append(int(rng.integers(0, 5))); W.append(0.0); P.append(1.0 / 3); cb.append(0); cc.append(0); act.append(j)
        N[spine] = max(N[spine], sum(N[first:first + fan]) + 1)
        spine = first + nxt
    soa = dict(N=np.array(N, np.int32), W=np.array(W, np.float32), P=np.array(P, np.float32),
               VL=np.zeros(len(N), np.int32), child_begin=np.array(cb, np.int32), child_count=np.array(cc, np.int32),
               action=np.array(act, np.int32))
    return soa


@pytest.mark.parametrize("dominate,fan,B", [(True, 5, 700), (True, 70, 900), (False, 9, 1000), (True, 5, 30)])
def test_long_chains_of_crowded_nodes(dominate, fan, B):
    # level after level the owner wavefront walks on into the kept child while a helper shares
    # out the visitors of the node before; the spine ends in a leaf right after such a hand-over
    soa = chain_forest(11, 40, fan, dominate)
    st = select_both(soa, np.zeros(B, np.int32), 50, steps=3)
    assert st["replayed_nodes"] == 0, st


def dominated_forest(seed, fan, depth, rave, kind, visitors):
    """A chain of nodes in each of which ONE child takes nearly every visitor and a few others get a
    visit or two in between.  The dominant child scores 0.9 and loses about 1.1e-4 per visit; the
    rivals' first scores are placed in the band it sweeps with `visitors` visits.  kind "few" =
    rivals with few visits (one entry each gets in), "some" = rivals that hold out for several
    entries, "late" = a child whose score is mostly exploration shows the best first score of all
    and drops at once, "plateau" (RAVE) = rivals whose blended score hardly moves with virtual loss
    and that meet the dominant child near the end."""
    rng = np.random.default_rng(seed)
    N, W, P, cb, cc, act, rN, rW = ([] for _ in range(8))

    def add(n, w, p, a, rn=0, rw=0.0):
        N.append(int(n)); W.append(float(w)); P.append(float(p)); cb.append(0); cc.append(0); act.append(a)
        rN.append(int(rn)); rW.append(float(rw))
        return len(N) - 1

    fans = fan if isinstance(fan, (list, tuple)) else [fan]
    node = add(60_000, 0.0, 0.0, -1)
    for level in range(depth):
        fan = fans[level % len(fans)]
        ep = 1.4 * np.sqrt(N[node])
        cb[node] = len(N)
        cc[node] = fan
        dom = int(rng.integers(fan))
        kids = []
        for i in range(fan):
            n = int(rng.integers(5, 60))
            q = rng.uniform(-0.2, 0.5)
            rn = int(rng.integers(0, 30))
            kids.append(add(n, q * n, rng.uniform(1e-5, 2e-4), i, rn, rng.uniform(-0.5, 0.3) * rn))
        c = kids[dom]
        N[c] = 50_000; W[c] = 0.9 * 50_000; P[c] = 0.01; rN[c] = 600; rW[c] = 0.5 * 600
        swept = 1.1e-4 * visitors  # what the dominant child's score loses over the visits
        rivals = [k for k in rng.permutation(fan) if k != dom][:4]
        for j, k in enumerate(rivals):
            r = kids[k]
            target = 0.9 - swept * rng.uniform(0.1, 0.95)  # first score inside the band
            if kind == "late" and j == 0:
                N[r] = 3; W[r] = 1.0; P[r] = (0.97 - 1.0 / 3) * 4 / ep
            elif kind == "plateau" and j < 2:
                n, rn, rave_value = 40_000, 500, 0.45
                beta = np.sqrt(1000.0 / (3 * n + 1000.0))
                N[r] = n; W[r] = (target - beta * rave_value) / (1 - beta) * n; P[r] = 1e-6; rN[r] = rn; rW[r] = rave_value * rn
            elif kind == "some":
                N[r] = 3000; W[r] = 0.85 * 3000; P[r] = (target - 0.85) * 3001 / ep
            else:
                N[r] = 30; W[r] = 0.6 * 30; P[r] = (target - 0.6) * 31 / ep
        node = c
    soa = dict(N=np.array(N, np.int32), W=np.array(W, np.float32), P=np.array(P, np.float32),
               VL=np.zeros(len(N), np.int32), child_begin=np.array(cb, np.int32), child_count=np.array(cc, np.int32),
               action=np.array(act, np.int32))
    if rave:
        soa["rN"] = np.array(rN, np.int32)
        soa["rW"] = np.array(rW, np.float32)
    return soa


@pytest.mark.parametrize("visitors", [9, 40, 200, 900])
@pytest.mark.parametrize("fan,rave,kind", [(40, False, "few"), (40, False, "some"), (40, False, "late"),
                                           (362, True, "few"), (362, True, "late"), (362, True, "plateau"),
                                           (150, True, "plateau"), (150, True, "some")])
def test_one_child_takes_nearly_every_visitor(visitors, fan, rave, kind):
    """Nodes settled by merging the few entries of other children into the dominant child's list
    (no threshold search, no sort) give the serial order, for every way such a node comes about."""
    soa = dominated_forest(100 + visitors + fan, fan, 6, rave, kind, visitors)
    st = select_both(soa, np.zeros(visitors, np.int32), 8, rave=rave, steps=3)
    assert st["replayed_nodes"] == 0, st
    # (with plateau rivals the child that holds out longest takes over for good near the end, and
    # everything before that is "other children's entries": merged only while those are few)
    if kind != "plateau" or visitors <= 40:
        assert st["merged_nodes"] >= 1, st


@pytest.mark.parametrize("visitors", [40, 900])
@pytest.mark.parametrize("rave,kind", [(False, "few"), (True, "few"), (True, "plateau"), (False, "some")])
def test_chain_through_narrow_and_wide_nodes(rave, kind, visitors):
    """The crowd walks down a chain whose nodes change between the narrow class (at most 64 children, one
    wavefront loads them) and the wide one (three wavefronts share the children of the node the owner
    walks on into), in every order: narrow to wide, wide to narrow, wide to wider."""
    soa = dominated_forest(31, [40, 200, 64, 65, 362, 10, 130, 300, 300, 7], 20, rave, kind, visitors)
    st = select_both(soa, np.zeros(visitors, np.int32), 22, rave=rave, steps=3)
    assert st["replayed_nodes"] == 0, st



def capacity_chain(fan, depth, at, m, rave, seed=5):
    """A spine of `depth` nodes, every one of which sends all m visitors into its spine child, except the
    node at level `at`: there one sibling's prior is the smallest binary32 number with which it is chosen at
    all, found by bisection on the checker itself, so that the spine child's capacity (the visitors it
    takes before any other child gets one) is exactly m - 1: the LAST visitor leaves the spine."""
    rng = np.random.default_rng(seed)
    N, W, P, cb, cc, act, rN, rW = [10 ** 6], [0.0], [0.0], [0], [0], [-1], [0], [0.0]
    spine, special = 0, -1
    for d in range(depth):
        first = len(N)
        cb[spine], cc[spine] = first, fan
        nxt = int(rng.integers(fan))
        for i in range(fan):
            if i == nxt:
                N.append(100000); W.append(90000.0); P.append(0.9)
                rN.append(50); rW.append(40.0)
            else:
                n = int(rng.integers(1, 30))
                N.append(n); W.append(float(np.float32(-rng.uniform(0, n)))); P.append(0.1 / fan)
                rN.append(int(rng.integers(0, 9))); rW.append(float(np.float32(-rng.uniform(0, 3))))
            cb.append(0); cc.append(0); act.append(i)
        if d == at:
            special = first + (nxt + 1) % fan
            N[special], W[special], rN[special], rW[special] = 0, 0.0, 0, 0.0
        spine = first + nxt
    soa = dict(N=np.array(N, np.int32), W=np.array(W, np.float32), P=np.array(P, np.float32),
               VL=np.zeros(len(N), np.int32), child_begin=np.array(cb, np.int32), child_count=np.array(cc, np.int32),
               action=np.array(act, np.int32))
    if rave:
        soa["rN"], soa["rW"] = np.array(rN, np.int32), np.array(rW, np.float32)
    rp = R.make_params(c_puct=1.4, virtual_loss=3, use_rave=rave, rave_k=1000.0, max_depth=depth + 2)
    roots = np.zeros(m, np.int32)

    def taken(p):
        soa["P"][special] = p
        paths, plen, _, _ = R.RefTree.from_soa(soa).select_batch(roots, rp, near_ties=False)
        return np.nonzero(paths[:, at + 1] == special)[0]

    lo, hi = np.float32(0.0), np.float32(1.0)
    assert len(taken(lo)) == 0 and len(taken(hi)) > 0
    while np.nextafter(lo, np.float32(2.0)) < hi:
        mid = np.float32((np.float64(lo) + np.float64(hi)) / 2)
        if len(taken(mid)):
            hi = mid
        else:
            lo = mid
    who = taken(hi)
    assert who.tolist() == [m - 1], who       # the last visitor, and nobody else, leaves the spine at that level
    return soa


@pytest.mark.parametrize("fan,rave,m", [(40, False, 200), (300, True, 200), (362, False, 37), (9, True, 900)])
def test_chain_whose_capacity_is_exceeded_by_one_visitor(fan, rave, m):
    """25 nodes in a row whose visitors all follow one child; at the 12th the best child takes all visitors
    but the last one.  The walk down such nodes must stop exactly there, and hand the node over with
    the right verdict."""
    soa = capacity_chain(fan, 25, 11, m, rave)
    st = select_both(soa, np.zeros(m, np.int32), 27, rave=rave, steps=2)
    assert st["replayed_nodes"] == 0, st


def test_boundaries_of_heavy_children_are_worked_out_ahead_of_time():
    """A heavy root with heavy children: the children's slice boundaries are queued as items of their own
    (kind 4 in the timeline) while the root is still being settled, the root's own when the roots are set;
    the result is the checker's all the same, and nothing is replayed."""
    import omoknuni_small_amd as omk
    soa, roots = layered_forest(12, [48, 40])
    troots = np.zeros(20_000, np.int32)
    D, vl = 3, 3
    ref = R.RefTree.from_soa(soa)
    rp = R.make_params(c_puct=1.4, virtual_loss=vl, max_depth=D)
    f = omk.Forest.from_soa(soa)
    b = omk.Batch(f, len(troots), D)
    b.set_roots(troots)
    b.enable_stats()
    b.enable_trace()
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=vl)
    rpaths, rlen, rleaf, near = ref.select_batch(troots, rp)
    b.select(sp)
    tr = b.debug_trace()
    gpaths, glen, gleaf, _ = b.read()
    st = b.stats()
    assert (gpaths == rpaths).all() and (glen == rlen).all() and (gleaf == rleaf).all()
    assert st["replayed_nodes"] == 0, st
    kind = (tr[:, 2] >> 60) & 7
    depth = (tr[:, 2] >> 32) & 0xFFFFFFF
    assert ((kind == 4) & (depth == 0)).sum() >= 1, "no boundary of the root was queued"
    assert ((kind == 4) & (depth == 1)).sum() >= 1, "no boundary of a heavy child was queued ahead of time"
    assert (kind == 1).sum() >= 1


def test_roots_set_again_start_the_paths_anew():
    """The paths' first entries are written when the roots are set: setting other roots replaces them."""
    import omoknuni_small_amd as omk
    soa, roots = layered_forest(13, [30, 10], n_trees=4)
    f = omk.Forest.from_soa(soa)
    b = omk.Batch(f, 600, 3)
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=3)
    for pick in ([0, 1], [2, 3, 1], [3]):
        troots = roots[np.array(pick)][np.arange(600) % len(pick)].astype(np.int32)
        ref = R.RefTree.from_soa(soa)
        rp = R.make_params(c_puct=1.4, virtual_loss=3, max_depth=3)
        rpaths, rlen, rleaf, _ = ref.select_batch(troots, rp)
        b.set_roots(troots)
        b.select(sp)
        gpaths, glen, gleaf, _ = b.read()
        assert (gpaths[:, 0] == troots).all()
        assert (gpaths == rpaths).all() and (glen == rlen).all() and (gleaf == rleaf).all()
        f.upload(soa)  # the virtual losses of this selection are dropped with the statistics


def test_call_numbers_start_over_without_a_trace():
    """The queues' ready marks are call numbers, which start over shortly before 2^30 calls (all marks, the
    boundary table and the heavy nodes' contexts cleared): selections on both sides of that point, with heavy
    nodes, slices, boundaries worked out ahead of time, lone walkers and the depth-cap counter, stay exact."""
    import omoknuni_small_amd as omk
    soa, roots = layered_forest(21, [150, 30, 6], n_trees=2)
    B, D, vl = 9000, 3, 3              # the depth bound cuts every path at a node with children
    troots = roots[np.sort(np.arange(B) % 2)].astype(np.int32)
    ref = R.RefTree.from_soa(soa)
    rp = R.make_params(c_puct=1.4, virtual_loss=vl, max_depth=D)
    f = omk.Forest.from_soa(soa)
    b = omk.Batch(f, B, D)
    b.set_roots(troots)
    b.enable_stats()
    sp = omk.SelectParams(c_puct=1.4, virtual_loss=vl)
    rng = np.random.default_rng(2)
    sliced = 0
    for step in range(10):
        if step == 2:
            b.debug_set_select_count((1 << 30) - 6)       # four calls before the numbers start over
        rpaths, rlen, rleaf, _ = ref.select_batch(troots, rp, near_ties=False)
        b.select(sp)
        gpaths, glen, gleaf, _ = b.read()
        assert (gpaths == rpaths).all() and (glen == rlen).all() and (gleaf == rleaf).all(), step
        assert b.truncated() == int(((ref.child_count[rleaf] > 0) & (rlen == D + 1)).sum()), step
        sliced += b.stats()["sliced_nodes"]
        vals = rng.uniform(-1, 1, B).astype(np.float32)
        ref.backup_batch(rpaths, rlen, vals, vl)
        b.set_values(vals)
        b.backup(vl)
        st = f.download()
        assert (st["N"] == ref.N).all() and (st["VL"] == ref.VL).all(), step
        ref.W[:] = st["W"]
    assert sliced >= 10
    with pytest.raises(omk.OmkError):
        b.debug_set_select_count(1)                        # forward only
