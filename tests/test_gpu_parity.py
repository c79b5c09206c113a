"""GPU parity: the HIP path, called through the C ABI, against the CPU checker on the same
seeded trees.  Bar: selected children, paths, path lengths, leaves, move lists, N and
virtual-loss counters bit-exact; W within 1e-5 relative (float atomics reorder the sums).
Selections whose top-2 scores lie within 1e-6 relative are reported separately: a
mismatch is only tolerated on a traversal the checker flagged as such a near tie."""
import numpy as np
import pytest

from oracle import ref_cpu as R
from tests.helpers import random_tree, star

pytestmark = pytest.mark.gpu

W_RTOL = 1e-5


def _gpu():
    import omoknuni_small_amd as omk
    return omk


def run_both(soa, roots, B_roots, c_puct=1.4, vl=3, use_rave=False, rave_k=1000.0, pw=False, max_depth=8,
             values_seed=0, do_backup=True):
    omk = _gpu()
    rp = R.make_params(c_puct=c_puct, virtual_loss=vl, use_rave=use_rave, rave_k=rave_k, pw=pw, max_depth=max_depth)
    ref = R.RefTree.from_soa(soa)
    rpaths, rlen, rleaf, near = ref.select_batch(B_roots, rp)
    ract = ref.gather_actions(rpaths, rlen)

    f = omk.Forest.from_soa(soa)
    b = omk.Batch(f, len(B_roots), max_depth)
    b.set_roots(B_roots)
    sp = omk.SelectParams(c_puct=c_puct, virtual_loss=vl, use_rave=use_rave, rave_k=rave_k, pw=pw)
    b.select(sp)
    gpaths, glen, gleaf, gact = b.read()
    after_select = f.download()

    bad = np.nonzero((gpaths != rpaths).any(axis=1) | (glen != rlen) | (gleaf != rleaf))[0]
    n_near = int((near >= 0).sum())
    if len(bad):
        not_near = [int(t) for t in bad if near[t] < 0]
        assert not not_near, "paths differ on traversals without a near tie: %s (near ties: %d)" % (not_near[:8], n_near)
        pytest.fail("paths differ only on %d near-tie traversals of %d flagged: reported separately" % (len(bad), n_near))
    assert (gact == ract).all()
    assert (after_select["VL"] == ref.VL).all(), "virtual loss after select"
    assert (after_select["N"] == ref.N).all()
    assert after_select["W"].tobytes() == ref.W.tobytes()

    if do_backup:
        values = np.random.default_rng(values_seed).uniform(-1, 1, len(B_roots)).astype(np.float32)
        ref.backup_batch(rpaths, rlen, values, vl)
        b.set_values(values)
        b.backup(vl)
        got = f.download()
        assert (got["N"] == ref.N).all(), "N after backup"
        assert (got["VL"] == ref.VL).all(), "virtual loss after backup"
        scale = np.maximum(np.abs(ref.W), 1.0)
        err = np.abs(got["W"].astype(np.float64) - ref.W.astype(np.float64)) / scale
        assert err.max() <= W_RTOL, "W after backup: max rel err %g" % err.max()
    b.close()
    f.close()
    return n_near


def test_known_answers_on_gpu(golden):
    omk = _gpu()
    for k in golden["select"]:
        rave = "rave" in k
        soa = star(k["Np"], k["children"], rave=rave)
        f = omk.Forest.from_soa(soa)
        b = omk.Batch(f, 1, 1)
        b.set_roots([0])
        b.select(omk.SelectParams(c_puct=k["c"], virtual_loss=0))
        _, _, leaf, _ = b.read()
        assert leaf[0] - 1 == k["plain"], k["id"]
        if rave:
            b.select(omk.SelectParams(c_puct=k["c"], virtual_loss=0, use_rave=True, rave_k=k["rave_k"]))
            _, _, leaf, _ = b.read()
            assert leaf[0] - 1 == k["rave"], k["id"]
        b.close()
        f.close()


def test_known_answer_backup_on_gpu(golden):
    omk = _gpu()
    k = golden["backup"][0]
    nd = k["nodes"]
    order = ["root", "a", "b", "c"]
    soa = dict(N=np.array([nd[x][0] for x in order], np.int32), W=np.array([nd[x][1] for x in order], np.float32),
               P=np.array([0, 1, 1, 1], np.float32), VL=np.zeros(4, np.int32),
               child_begin=np.array([1, 2, 3, 0], np.int32), child_count=np.array([1, 1, 1, 0], np.int32))
    f = omk.Forest.from_soa(soa)
    b = omk.Batch(f, 1, 8)
    b.set_roots([0])
    b.select(omk.SelectParams(virtual_loss=k["virtual_loss"]))
    paths, plen, leaf, act = b.read()
    assert list(paths[0, :4]) == [0, 1, 2, 3] and plen[0] == 4 and leaf[0] == 3
    assert list(f.download()["VL"]) == k["post_select_vl"]
    b.set_values([k["leaf_value"]])
    b.backup(k["virtual_loss"])
    got = f.download()
    for i, x in enumerate(order):
        n, w, vl = k["post_backup"][x]
        assert got["N"][i] == n and got["VL"][i] == vl
        assert got["W"][i] == pytest.approx(w, rel=1e-6)


@pytest.mark.parametrize("seed", range(6))
def test_small_fanout_single_tree(seed):
    soa, roots = random_tree(seed, n_expand=60, fanout=(1, 12), max_depth=6, tie_frac=0.2, vl_frac=0.1)
    run_both(soa, roots, np.zeros(48, np.int32), max_depth=8, values_seed=seed)


@pytest.mark.parametrize("seed,fan", [(10, (40, 64)), (11, (65, 130)), (12, (200, 256)), (13, (300, 384)),
                                      (14, (500, 1024)), (15, (1, 400))])
def test_wide_fanout(seed, fan):
    soa, roots = random_tree(seed, n_expand=25, fanout=fan, max_depth=5, zero_frac=0.5, tie_frac=0.1)
    run_both(soa, roots, np.zeros(200, np.int32), max_depth=6, values_seed=seed)


@pytest.mark.parametrize("seed", [20, 21, 22])
def test_legal_mask(seed):
    soa, roots = random_tree(seed, n_expand=40, fanout=(20, 230), max_depth=5, mask_frac=0.5)
    run_both(soa, roots, np.zeros(128, np.int32), max_depth=6, values_seed=seed)


@pytest.mark.parametrize("seed", [30, 31, 32])
def test_rave_two_pass(seed):
    soa, roots = random_tree(seed, n_expand=40, fanout=(2, 90), max_depth=5, rave=True, zero_frac=0.4)
    run_both(soa, roots, np.zeros(96, np.int32), use_rave=True, rave_k=1000.0, max_depth=6, values_seed=seed)
    run_both(soa, roots, np.zeros(96, np.int32), use_rave=True, rave_k=3000.0, c_puct=0.3, max_depth=6)


@pytest.mark.parametrize("visitors", [1, 3, 40, 1500])
def test_rave_second_scan_needs_a_first_scan_winner(visitors):
    """Every first-scan score is NaN (unvisited children under virtual loss whose value sum is NaN)
    while the RAVE blend of the second scan is finite: the reference skips the second scan and falls
    back to the least-visited child, first minimum (mcts_node.cpp:173-184), for every visitor."""
    kids = [[0, float("nan"), 0.2, 2, 5 + i, float(i)] for i in range(70)]
    soa = star(10, kids, rave=True)
    # one level further down the same situation among visited children (N > 0, W = NaN)
    base = len(soa["N"])
    extra = 5
    soa["child_begin"][1] = base
    soa["child_count"][1] = extra
    app = lambda key, vals, dt: np.concatenate([soa[key], np.asarray(vals, dt)])
    soa["N"] = app("N", [4, 2, 9, 2, 7], np.int32)
    soa["W"] = app("W", [float("nan")] * extra, np.float32)
    soa["P"] = app("P", [0.2] * extra, np.float32)
    soa["VL"] = app("VL", [0] * extra, np.int32)
    soa["rN"] = app("rN", [3, 3, 3, 3, 3], np.int32)
    soa["rW"] = app("rW", [1.0, 2.0, 3.0, -1.0, 0.5], np.float32)
    soa["child_begin"] = app("child_begin", [0] * extra, np.int32)
    soa["child_count"] = app("child_count", [0] * extra, np.int32)
    soa["action"] = app("action", list(range(extra)), np.int32)
    ref = R.RefTree.from_soa(soa)
    rp = R.make_params(use_rave=True, rave_k=1000.0, max_depth=3)
    assert ref.select_child(0, rp) == 1 and ref.select_child(1, rp) == base + 1  # least visited, first minimum
    # no backup: the value sums are NaN on purpose, which the W comparison cannot take
    run_both(soa, np.array([0], np.int32), np.zeros(visitors, np.int32), use_rave=True, rave_k=1000.0, max_depth=3,
             do_backup=False)


@pytest.mark.parametrize("seed", [40, 41])
def test_forest_of_trees(seed):
    soa, roots = random_tree(seed, n_expand=120, fanout=(3, 70), max_depth=6, n_roots=8)
    rng = np.random.default_rng(seed)
    B_roots = roots[rng.integers(0, len(roots), 300)]  # interleaved, unsorted tree ids
    run_both(soa, roots, B_roots.astype(np.int32), max_depth=7, values_seed=seed)


@pytest.mark.parametrize("vl", [0, 1, 3, 7])
def test_virtual_loss_amounts(vl):
    soa, roots = random_tree(50 + vl, n_expand=50, fanout=(2, 40), max_depth=6, vl_frac=0.3)
    run_both(soa, roots, np.zeros(150, np.int32), vl=vl, max_depth=7, values_seed=vl)


def test_progressive_widening_sorted():
    soa, roots = random_tree(60, n_expand=60, fanout=(1, 150), max_depth=6, sort_prior=True, n_max=400)
    run_both(soa, roots, np.zeros(256, np.int32), pw=True, max_depth=7)


def test_depth_cap_truncates():
    omk = _gpu()
    soa, roots = random_tree(70, n_expand=80, fanout=(1, 3), max_depth=12)
    n_near = run_both(soa, roots, np.zeros(32, np.int32), max_depth=3)
    f = omk.Forest.from_soa(soa)
    b = omk.Batch(f, 32, 3)
    b.set_roots(np.zeros(32, np.int32))
    b.select(omk.SelectParams())
    _, plen, leaf, _ = b.read()
    expect = int(((plen == 4) & (soa["child_count"][leaf] > 0)).sum())
    assert b.truncated() == expect
    assert n_near >= 0


def test_depth_cap_counter_over_consecutive_selects():
    """The count of depth-capped simulations is per select, whichever launches the select consists of:
    lone traversals (one launch, no reset before it) twice in a row, then traversals that share
    roots, then lone ones again."""
    omk = _gpu()
    soa, roots = random_tree(71, n_expand=120, fanout=(2, 4), max_depth=10, n_roots=6)
    f = omk.Forest.from_soa(soa)
    b = omk.Batch(f, 24, 2)
    sp = omk.SelectParams(virtual_loss=0)

    def run(troots):
        b.set_roots(np.asarray(troots, np.int32))
        b.select(sp)
        _, plen, leaf, _ = b.read()
        expect = int(((plen == 3) & (soa["child_count"][leaf] > 0)).sum())
        assert expect > 0
        assert b.truncated() == expect
        return expect

    alone = run(roots)
    assert run(roots) == alone
    run(np.repeat(roots, 4))
    assert run(roots) == alone
    run(roots[:3])


def test_all_equal_scores_tie_to_lowest_index():
    # unvisited children with equal priors: every pick is an exact tie until virtual loss separates them
    k = 300
    soa = star(0, [[0, 0.0, 1.0 / k, 0]] * k)
    soa["N"][0] = 17
    run_both(soa, np.array([0]), np.zeros(700, np.int32), max_depth=2)


def test_nan_scores_fall_back_to_least_visited():
    soa = star(10, [[5, np.nan, .2, 0], [3, np.nan, .2, 0], [3, np.nan, .2, 0], [9, np.nan, .4, 0]])
    run_both(soa, np.array([0]), np.zeros(5, np.int32), max_depth=2, do_backup=False)


def test_revert_then_backup_without_virtual_loss():
    """apply (inside select), explicit revert, then backup with amount 0: the three separate steps."""
    omk = _gpu()
    soa, roots = random_tree(80, n_expand=60, fanout=(2, 50), max_depth=6)
    B_roots = np.zeros(200, np.int32)
    rp = R.make_params(virtual_loss=3, max_depth=7)
    ref = R.RefTree.from_soa(soa)
    rpaths, rlen, _, _ = ref.select_batch(B_roots, rp)
    ref.revert_vl_paths(rpaths, rlen, 3)
    f = omk.Forest.from_soa(soa)
    b = omk.Batch(f, 200, 7)
    b.set_roots(B_roots)
    b.select(omk.SelectParams(virtual_loss=3))
    b.revert_vl(3)
    assert (f.download()["VL"] == ref.VL).all()
    values = np.random.default_rng(1).uniform(-1, 1, 200).astype(np.float32)
    ref.backup_batch(rpaths, rlen, values, 0)
    b.set_values(values)
    b.backup(0)
    got = f.download()
    assert (got["N"] == ref.N).all() and (got["VL"] == ref.VL).all()
    assert np.allclose(got["W"], ref.W, rtol=W_RTOL, atol=W_RTOL)


def test_path_kernels_on_arbitrary_paths():
    """The atomic apply / revert / backup entry points over caller-built paths, with nodes shared
    between paths at unrelated depths and pre-existing virtual loss."""
    omk = _gpu()
    rng = np.random.default_rng(5)
    n_nodes, B, L = 500, 333, 9
    soa = dict(N=rng.integers(0, 50, n_nodes).astype(np.int32), W=rng.uniform(-5, 5, n_nodes).astype(np.float32),
               P=np.zeros(n_nodes, np.float32), VL=rng.integers(0, 12, n_nodes).astype(np.int32),
               child_begin=np.zeros(n_nodes, np.int32), child_count=np.zeros(n_nodes, np.int32))
    plen = rng.integers(1, L + 1, B).astype(np.int32)
    rows = rng.integers(0, n_nodes, (B, L)).astype(np.int32)
    rows[:, 0] = 7  # a shared root
    values = rng.uniform(-1, 1, B).astype(np.float32)
    stride = 384
    lm = np.full((L, stride), -1, np.int32)
    lm[:, :B] = rows.T
    f = omk.Forest.from_soa(soa)
    d_paths, d_len, d_val = f.dev_alloc(lm.nbytes), f.dev_alloc(plen.nbytes), f.dev_alloc(values.nbytes)
    f.h2d(d_paths, lm)
    f.h2d(d_len, plen)
    f.h2d(d_val, values)
    ref = R.RefTree.from_soa(soa)
    for amount in (3, 1):
        ref.apply_vl_paths(rows, plen, amount)
        f.apply_vl_paths(d_paths, d_len, B, stride, L, amount)
        assert (f.download()["VL"] == ref.VL).all(), "apply"
    ref.revert_vl_paths(rows, plen, 2)
    f.revert_vl_paths(d_paths, d_len, B, stride, L, 2)
    assert (f.download()["VL"] == ref.VL).all(), "revert"
    for amount in (3, 0):
        ref.backup_batch(rows, plen, values, amount)
        f.backup_paths(d_paths, d_len, d_val, B, stride, L, amount)
        got = f.download()
        assert (got["N"] == ref.N).all() and (got["VL"] == ref.VL).all(), "backup amount %d" % amount
        assert np.allclose(got["W"], ref.W, rtol=W_RTOL, atol=1e-4)
    for p in (d_paths, d_len, d_val):
        f.dev_free(p)


def test_transposition_table_matches_checker_and_dict():
    omk = _gpu()
    rng = np.random.default_rng(9)
    log2 = 12
    n_ins = 1 << (log2 - 1)  # 50 % load
    keys = rng.integers(0, 2**63, n_ins, dtype=np.uint64)
    keys[:64] = (np.arange(64, dtype=np.uint64) << np.uint64(52))  # shared home slots: long probe chains
    keys = np.unique(keys)
    rng.shuffle(keys)
    nodes = rng.integers(0, 10**6, len(keys)).astype(np.int32)
    depths = rng.integers(0, 6, len(keys)).astype(np.int32)
    soa = star(1, [[0, 0, 1, 0]])
    f = omk.Forest.from_soa(soa)
    tt = omk.TranspositionTable(f, log2)
    tt.insert(keys, nodes, depths)
    ref = R.RefTT(log2)
    for k, n, d in zip(keys, nodes, depths):
        assert ref.insert(k, n, d) == 0
    probe = np.concatenate([keys[: len(keys) // 2], rng.integers(0, 2**63, 3000, dtype=np.uint64)])
    table = {int(k): (int(n), int(d)) for k, n, d in zip(keys, nodes, depths)}
    for min_depth in (0, 3):
        got = tt.probe(probe, min_depth)
        want, _ = ref.probe(probe, min_depth)
        brute = np.array([table[int(k)][0] if int(k) in table and table[int(k)][1] >= min_depth else -1
                          for k in probe], np.int32)
        assert (want == brute).all()
        assert (got == brute).all()
    # the device-built table holds the same set of entries as the serially built one
    dev = tt.download()
    occ = dev[dev["key"] != np.uint64(2**64 - 1)]
    assert len(occ) == len(keys)
    assert set(map(int, occ["key"])) == set(map(int, keys))
    # serial table uploaded as is gives the same answers
    tt.upload(ref.slots)
    assert (tt.probe(probe, 0) == ref.probe(probe, 0)[0]).all()
    # second insert of present keys keeps the first entry
    tt.insert(keys[:100], np.full(100, -5, np.int32))
    assert (tt.probe(keys[:100]) == nodes[:100]).all()


def test_error_paths_do_not_reach_the_device():
    omk = _gpu()
    soa = star(3, [[1, 0.5, .5, 0], [1, 0.1, .5, 0]])
    bad = dict(soa)
    bad["child_begin"] = soa["child_begin"].copy()
    bad["child_begin"][0] = 2  # range runs past the end
    with pytest.raises(omk.OmkError) as e:
        omk.Forest.from_soa(bad)
    assert e.value.code == -4
    dag = dict(soa)
    dag["child_begin"] = np.array([1, 2, 0], np.int32)
    dag["child_count"] = np.array([2, 1, 0], np.int32)  # node 2 has two parents
    with pytest.raises(omk.OmkError):
        omk.Forest.from_soa(dag)
    f = omk.Forest.from_soa(soa)
    b = omk.Batch(f, 4, 2)
    with pytest.raises(omk.OmkError):
        b.set_roots([5])
    with pytest.raises(omk.OmkError):
        b.backup(3)  # nothing selected yet
    b.set_roots([0, 0])
    with pytest.raises(omk.OmkError):
        b.select(omk.SelectParams(use_rave=True))  # forest has no RAVE arrays
