"""The compaction entry point that allocates nothing (omk_forest_compact_static: all its device
scratch memory is one array inside the library) against omk_forest_compact on the same forests, two
calls in a row, the second on a smaller input; everything through the C ABI."""
import numpy as np
import pytest

from oracle import ref_cpu as R
from tests.helpers import random_tree

pytestmark = pytest.mark.gpu


def _most_visited_child(soa, root):
    kids = np.arange(soa["child_begin"][root], soa["child_begin"][root] + soa["child_count"][root])
    if "legal" in soa:
        kids = kids[((soa["legal"][kids >> 5] >> (kids & 31).astype(np.uint32)) & 1) == 1]
    return int(kids[np.argmax(soa["N"][kids])])


def _same(a, b, what):
    sa, sb = a.download(), b.download()
    assert a.node_count()[0] == b.node_count()[0], what
    for k in sa:
        assert sa[k].tobytes() == sb[k].tobytes(), "%s: %s differs" % (what, k)
    ta, tb = a.download_structure(), b.download_structure()
    for k in ta:
        assert (ta[k] == tb[k]).all(), "%s: %s differs" % (what, k)


def _forest_pair(omk, soa):
    return omk.Forest.from_soa(soa), omk.Forest.from_soa(soa)


@pytest.mark.parametrize("mask_frac,rave", [(0.0, False), (0.25, True)])
def test_static_compaction_matches_the_allocating_one(mask_frac, rave):
    import omoknuni_small_amd as omk
    big, roots_big = random_tree(71, n_expand=900, fanout=(2, 30), max_depth=9, mask_frac=mask_frac, rave=rave, n_max=500)
    small, roots_small = random_tree(72, n_expand=60, fanout=(1, 9), max_depth=5, mask_frac=mask_frac, rave=rave, n_max=80)
    # two calls in a row on one GPU, the second with a smaller input: what the first left in the
    # shared scratch memory must not show
    for soa, roots, tag in ((big, roots_big, "first call"), (small, roots_small, "second, smaller call")):
        fa, fs = _forest_pair(omk, soa)
        child = _most_visited_child(soa, int(roots[0]))
        oa = fa.compact(child)
        os_ = fs.compact(child, static=True)
        assert (oa == os_).all(), tag
        _same(fa, fs, tag)
        ref2, order = R.RefTree.from_soa(soa).compacted(child)
        assert (os_ == order).all() and fs.node_count()[0] == ref2.n, tag
        # and once more on the result, smaller again: the subtree of its own most visited child
        st = fs.download_structure()
        cur = dict(fs.download(), **st)
        if "legal" in soa:
            bits = (soa["legal"][order >> 5] >> (order & 31).astype(np.uint32)) & 1
            pad = np.zeros((len(order) + 31) // 32 * 32, np.uint8)
            pad[:len(order)] = bits
            cur["legal"] = np.packbits(pad.reshape(-1, 32), axis=1, bitorder="little").view("<u4").reshape(-1).copy()
        if cur["child_count"][0] > 0:
            child2 = _most_visited_child(cur, 0)
            assert (fa.compact(child2) == fs.compact(child2, static=True)).all(), tag + " (again)"
            _same(fa, fs, tag + " (again)")
        # the compacted forest searches like the checker's
        B, D = 300, 9
        b = omk.Batch(fs, B, D)
        b.set_roots(np.zeros(B, np.int32))
        b.select(omk.SelectParams(c_puct=1.4, virtual_loss=3, use_rave=rave, rave_k=1000.0))
        b2 = omk.Batch(fa, B, D)
        b2.set_roots(np.zeros(B, np.int32))
        b2.select(omk.SelectParams(c_puct=1.4, virtual_loss=3, use_rave=rave, rave_k=1000.0))
        pa, ps = b2.read(), b.read()
        assert all((x == y).all() for x, y in zip(pa, ps)), tag


def test_static_compaction_refuses_what_does_not_fit():
    import omoknuni_small_amd as omk
    n = (1 << 20) + 1
    soa = dict(N=np.ones(n, np.int32), W=np.zeros(n, np.float32), P=np.zeros(n, np.float32), VL=np.zeros(n, np.int32),
               child_begin=np.zeros(n, np.int32), child_count=np.zeros(n, np.int32))
    soa["child_begin"][0], soa["child_count"][0] = 1, 3
    f = omk.Forest.from_soa(soa)
    with pytest.raises(omk.OmkError) as e:
        f.compact(1, static=True)
    assert e.value.code == -3 and "1048576" in str(e.value)  # OMK_ERR_CAPACITY, names the limit
    assert f.node_count()[0] == n  # nothing changed
    assert len(f.compact(0)) == 4  # the allocating entry point takes it
    assert len(f.compact(0, static=True)) == 4  # and now it fits
