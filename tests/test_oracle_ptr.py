"""The pointer-tree flavour of the checker (oracle/ref_ptr.cpp: the reference's node layout and
OpenMP loops, used for the timed CPU baseline) against the array checker: with one thread the
traversals run in index order, so paths and statistics must be identical."""
import numpy as np
import pytest

from oracle import ref_cpu as R
from oracle import ref_ptr as RP
from tests.helpers import random_tree


@pytest.mark.parametrize("seed,rave,mask", [(1, False, 0.0), (2, True, 0.0), (3, False, 0.3), (4, True, 0.3)])
def test_one_thread_matches_the_array_checker(seed, rave, mask):
    soa, roots = random_tree(seed, n_expand=150, fanout=(1, 30), max_depth=7, rave=rave, mask_frac=mask, vl_frac=0.2,
                             tie_frac=0.1, n_max=300)
    B, D, vl = 700, 9, 3
    troots = np.full(B, roots[0], np.int32)
    ref = R.RefTree.from_soa(soa)
    rp = R.make_params(c_puct=1.4, virtual_loss=vl, use_rave=rave, rave_k=500.0, max_depth=D)
    pt = RP.PtrTree(soa)
    rng = np.random.default_rng(seed)
    for step in range(3):
        values = rng.uniform(-1, 1, B).astype(np.float32)
        rpaths, rlen, rleaf, _ = ref.select_batch(troots, rp)
        ref.backup_batch(rpaths, rlen, values, vl)
        ppaths, plen, _, _ = pt.step(troots, values, virtual_loss=vl, use_rave=rave, rave_k=500.0, max_depth=D)
        assert (plen == rlen).all() and (ppaths == rpaths).all(), "step %d" % step
        st = pt.download()
        assert (st["N"] == ref.N).all() and (st["VL"] == ref.VL).all()
        assert (st["W"] == ref.W).all()  # same additions in the same order
    pt.close()


def test_node_record_is_as_large_as_the_reference_layout_implies():
    # five atomics on a cache line each plus the vector, prior, action: at least 6 lines
    assert RP.PtrTree.node_bytes() >= 6 * 64


def test_several_threads_finish_every_traversal():
    soa, roots = random_tree(9, n_expand=100, fanout=(2, 20), max_depth=6, n_max=100)
    B, D = 2000, 8
    pt = RP.PtrTree(soa)
    values = np.zeros(B, np.float32)
    paths, plen, _, _ = pt.step(np.full(B, roots[0], np.int32), values, max_depth=D, threads=4)
    st = pt.download()
    assert (plen >= 1).all() and (paths[:, 0] == roots[0]).all()
    assert (st["VL"] == 0).all()                       # every virtual loss reverted
    assert st["N"][roots[0]] == soa["N"][roots[0]] + B  # every traversal backed up through the root
    pt.close()
