"""The C++ host adapter (omk::ForestEngine, omoknuni_small_amd/csrc/omk_engine.h) driven like
the reference's search loop: batches of select -> evaluator -> backup."""
import os
import subprocess

import numpy as np
import pytest

from oracle import ref_cpu as R
from tests.helpers import random_tree

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "omoknuni_small_amd", "engine_smoke")


def write_forest(path, soa):
    with open(path, "wb") as f:
        f.write(np.int64(len(soa["N"])).tobytes())
        for k, dt in (("N", np.int32), ("W", np.float32), ("P", np.float32), ("VL", np.int32),
                      ("child_begin", np.int32), ("child_count", np.int32), ("action", np.int32)):
            f.write(np.ascontiguousarray(soa[k], dtype=dt).tobytes())


def evaluator(leaf, moves):
    h = np.int32(np.int32(leaf) * np.int32(31) + np.int32(len(moves)))
    with np.errstate(over="ignore"):
        for a in moves:
            h = np.int32(h * np.int32(17) + np.int32(a))
    h = int(h)
    r = h % 2001 if h >= 0 else -((-h) % 2001)  # C remainder
    return np.float32(np.float32(((r + 2001) % 2001) - 1000) / np.float32(1000.0))


def test_adapter_reports_errors_without_a_gpu(tmp_path):
    assert os.path.exists(EXE), "build the adapter first (python -m omoknuni_small_amd.build)"
    soa, _ = random_tree(1, n_expand=5)
    p = tmp_path / "f.bin"
    write_forest(p, soa)
    r = subprocess.run([EXE, str(p), "8", "4", "6"], capture_output=True, text=True, timeout=120)
    if r.returncode == 1:
        assert "engine error" in r.stderr and "omk_forest_create" in r.stderr  # no device: an exception, no crash
    else:
        assert r.returncode == 0


@pytest.mark.gpu
def test_adapter_search_loop_matches_checker(tmp_path):
    soa, _ = random_tree(7, n_expand=120, fanout=(2, 40), max_depth=8, n_max=200)
    p = tmp_path / "f.bin"
    write_forest(p, soa)
    sims, batch, D = 150, 64, 10
    r = subprocess.run([EXE, str(p), str(sims), str(batch), str(D)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().split("\n")
    assert lines[0] == "done %d leaves %d" % (sims, sims)
    got = np.array([[float(x) for x in ln.split()] for ln in lines[1:]])
    ref = R.RefTree.from_soa(soa)
    rp = R.make_params(c_puct=1.4, virtual_loss=3, max_depth=D)
    done = 0
    while done < sims:
        n = min(batch, sims - done)
        paths, plen, leaf, _ = ref.select_batch(np.zeros(n, np.int32), rp)
        acts = ref.gather_actions(paths, plen)
        vals = np.array([evaluator(leaf[i], list(acts[i, : plen[i] - 1])) for i in range(n)], np.float32)
        ref.backup_batch(paths, plen, vals, 3)
        done += n
    assert (got[:, 0] == ref.N).all() and (got[:, 2] == ref.VL).all()
    assert np.allclose(got[:, 1], ref.W, rtol=1e-5, atol=1e-5)


def leaf_hash(leaf, moves):
    h = np.int32(np.int32(leaf) * np.int32(31) + np.int32(len(moves)))
    with np.errstate(over="ignore"):
        for a in moves:
            h = np.int32(h * np.int32(17) + np.int32(a))
    return int(h) & 0xFFFFFFFF


@pytest.mark.gpu
def test_adapter_search_loop_with_expansion_matches_checker(tmp_path):
    """select -> evaluator -> expand -> backup, the tree growing on the device; the stand-in
    rules and policy of tests/cpp/engine_smoke.cpp restated here for the checker."""
    soa, _ = random_tree(9, n_expand=30, fanout=(2, 9), max_depth=4, n_max=60)
    p = tmp_path / "f.bin"
    write_forest(p, soa)
    sims, batch, D, A = 400, 50, 12, 8
    r = subprocess.run([EXE, str(p), str(sims), str(batch), str(D), "grow"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().split("\n")
    ref = R.RefTree.from_soa(soa)
    rp = R.make_params(c_puct=1.4, virtual_loss=3, max_depth=D)
    done = 0
    while done < sims:
        n = min(batch, sims - done)
        paths, plen, leaf, _ = ref.select_batch(np.zeros(n, np.int32), rp)
        acts = ref.gather_actions(paths, plen)
        seqs = [list(acts[i, : plen[i] - 1]) for i in range(n)]
        vals = np.array([evaluator(leaf[i], seqs[i]) for i in range(n)], np.float32)
        begin, moves = [0], []
        policy = np.zeros((n, A), np.float32)
        for i in range(n):
            h = leaf_hash(leaf[i], seqs[i])
            if h % 7 != 0:
                moves.extend((h + 3 * a) % 10 for a in range(1 + h % 4))
            begin.append(len(moves))
            for a in range(A):
                policy[i, a] = np.float32(np.float32((h + 5 * a) % 13) / np.float32(10.0)) - np.float32(0.1)
        ref.expand_batch(leaf, begin, moves, policy=policy, action_space=A)
        ref.backup_batch(paths, plen, vals, 3)
        done += n
    assert lines[0] == "done %d leaves %d nodes %d" % (sims, sims, ref.n)
    got = np.array([[float(x) for x in ln.split()] for ln in lines[1:]])
    assert len(got) == ref.n and ref.n > len(soa["N"])
    assert (got[:, 0] == ref.N).all() and (got[:, 2] == ref.VL).all()
    assert np.allclose(got[:, 1], ref.W, rtol=1e-5, atol=1e-5)
    assert (got[:, 3].astype(np.float32) == ref.P).all()
    assert (got[:, 4] == ref.child_begin).all() and (got[:, 5] == ref.child_count).all()
    assert (got[:, 6] == ref.action).all()
