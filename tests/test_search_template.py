"""omk::GPUForestMCTSEngine<State> (csrc/omk_search.h): MCTSEngine::search over the device forest with
the reference's signatures (search(const State&) -> SearchResult, an InferenceFunction over
unique_ptr<State> batches, leaf states built by clone + replay), driven by tests/cpp/search_smoke.cpp
with a mock state, and omk::flattenTree.  The whole search is replayed here through the CPU checker,
with the mock game and the stand-in evaluator restated in Python: every node of the final tree,
the move probabilities and the move chosen must come out the same."""
import os
import subprocess

import numpy as np
import pytest

from oracle import ref_cpu as R

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "omoknuni_small_amd", "search_smoke")
CELLS = 12


class Ring:
    """tests/cpp/search_smoke.cpp's RingState."""

    def __init__(self):
        self.cell = [0] * CELLS
        self.player, self.winner, self.moves = 1, 0, 0

    def clone(self):
        c = Ring()
        c.cell, c.player, c.winner, c.moves = list(self.cell), self.player, self.winner, self.moves
        return c

    def legal(self):
        return [i for i in range(CELLS) if self.cell[i] == 0] if self.winner == 0 else []

    def make(self, a):
        self.cell[a] = self.player
        if self.cell[(a + 1) % CELLS] == self.player and self.cell[(a - 1) % CELLS] == self.player:
            self.winner = self.player
        self.player = 3 - self.player
        self.moves += 1

    def terminal(self):
        return self.winner != 0 or self.moves == CELLS

    def hash(self):
        h = 1469598103934665603
        for c in self.cell:
            h = ((h ^ c) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
        return h ^ self.player


def evaluate(state):
    h = state.hash()
    value = np.float32(np.float32(int(h % 2001) - 1000) / np.float32(1000.0))
    pol = np.array([np.float32(1 + ((h >> (a * 3)) & 7)) for a in range(CELLS)], np.float32)
    s = np.float32(0.0)
    for x in pol:
        s = np.float32(s + x)
    return value, (pol / s).astype(np.float32)


class Mt19937:
    """Raw 32-bit outputs of std::mt19937(seed): numpy's legacy generator is the same engine with the same
    seeding, and a full-range draw returns its outputs one by one (5489 -> 3499211612 first)."""

    def __init__(self, seed):
        self.rs = np.random.RandomState(seed)

    def __call__(self):
        return int(self.rs.randint(0, 2 ** 32, dtype=np.uint64))


def shuffle_moves(moves, gen):
    """GPUForestMCTSEngine::shuffleMoves: Fisher-Yates from the last place down, j = output mod (k + 1)."""
    for k in range(len(moves) - 1, 0, -1):
        j = gen() % (k + 1)
        moves[k], moves[j] = moves[j], moves[k]
    return moves


def replay_search(sims, batch, widening, seed=5489, searches=1, follow=False):
    """`searches` searches one after the other on one engine (the generator of the shuffles runs on, the
    tree and the table of positions start empty every time: a table entry dies with the tree its node
    belongs to); the last one is returned."""
    gen = Mt19937(seed + 1)
    for _ in range(searches):
        ref = replay_one_search(sims, batch, widening, gen, follow)
    return ref


def replay_one_search(sims, batch, widening, gen, follow=False):
    root_state = Ring()
    root_state.make(3)
    z = np.zeros(1, np.int32)
    ref = R.RefTree(N=z, W=np.zeros(1, np.float32), P=np.ones(1, np.float32), VL=z, child_begin=z, child_count=z,
                    action=z - 1)
    rp = R.make_params(c_puct=1.4, virtual_loss=3, max_depth=16)
    # the table of positions: keys of the nodes from the game's own hash of the states they stand for,
    # known once a node has been a leaf; a node without a key is neither stored nor found
    table, key_of = R.RefTT(15), {}
    no_key = np.uint64(0xFFFFFFFFFFFFFFFF)
    entries = transpositions = 0
    done, first = 0, True
    # settings.follow_transpositions: the selection is the loop with the table, redirects included; every node
    # has its key from the moment it is created (keyNewChildren), and slots get re-pointed (alias)
    keys, alias = np.full(1, no_key, np.uint64), np.full(1, -1, np.int32)
    while done < sims:
        n = 1 if first else min(batch, sims - done)
        first = False
        roots = np.zeros(n, np.int32)
        if follow:
            grow = ref.n - len(keys)
            keys = np.concatenate([keys, np.full(grow, no_key, np.uint64)])
            alias = np.concatenate([alias, np.full(grow, -1, np.int32)])
            paths, plen, leaf, acts, counts = ref.select_redirect_batch(roots, rp, table, keys, alias)
            entries += int(counts[0])
            transpositions += int(counts[3])
        else:
            paths, plen, leaf, _ = ref.select_batch(roots, rp)
            acts = ref.gather_actions(paths, plen)
        begin, moves, pb, pol, values = [0], [], [0], [], []
        states = []
        for t in range(n):
            s = root_state.clone()
            for a in acts[t, :plen[t] - 1]:
                s.make(int(a))
            states.append(s)
            key_of[int(leaf[t])] = np.uint64(s.hash())
        if not follow:
            step_keys = np.array([[key_of.get(int(paths[t, d]), no_key) if d < plen[t] else no_key
                                   for d in range(1, paths.shape[1])] for t in range(n)], np.uint64).reshape(n, -1)
            _, counts = table.traverse(ref, paths, plen, step_keys)
            entries += counts[0]
            transpositions += counts[3]
        for t in range(n):
            s = states[t]
            v, p = evaluate(s)
            values.append(v)
            if not s.terminal():
                moves.extend(shuffle_moves(s.legal(), gen))   # the search shuffles as MCTSNode::expand does
            begin.append(len(moves))
            pol.extend(p.tolist())
            pb.append(len(pol))
        first_child = ref.expand_batch(leaf, begin, np.array(moves if moves else [0], np.int32),
                                       policy=np.array(pol, np.float32), action_space=CELLS, policy_begin=pb,
                                       widening=(2.0, 0.5) if widening else None)
        if follow:
            grow = ref.n - len(keys)
            keys = np.concatenate([keys, np.full(grow, no_key, np.uint64)])
            alias = np.concatenate([alias, np.full(grow, -1, np.int32)])
            for t in range(n):
                if first_child[t] >= 0:
                    for j in range(int(ref.child_count[leaf[t]])):
                        s = states[t].clone()
                        s.make(int(moves[begin[t] + j]))
                        keys[first_child[t] + j] = np.uint64(s.hash())
        ref.backup_batch(paths, plen, np.array(values, np.float32), 3)
        done += n
    ref.table_counts = (entries, transpositions)
    ref.alias = alias
    return ref


@pytest.mark.gpu
@pytest.mark.parametrize("widening", [0, 1])
def test_search_with_the_reference_signatures_matches_the_checker(widening):
    sims, batch = 300, 32
    r = subprocess.run([EXE, "search", str(sims), str(batch), str(widening), "0", "0"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().split("\n")
    head = lines[0].split()
    probs = np.array([float(x) for x in next(ln for ln in lines if ln.startswith("probabilities")).split()[1:]], np.float32)
    table = next(ln for ln in lines if ln.startswith("table entries")).split()
    nodes = np.array([[float(x) for x in ln.split()[2:]] for ln in lines if ln.startswith("node ")])
    ref = replay_search(sims, batch, widening)
    # the table of positions, keyed by the mock game's own getHash(): entries stored for unvisited children
    # and positions reached by another order of moves, as the checker counts them
    assert (int(table[2]), int(table[4])) == ref.table_counts, (table, ref.table_counts)
    assert ref.table_counts[0] > 0
    assert int(head[5]) == sims and int(head[7]) == ref.n == len(nodes) and int(head[9]) == sims
    assert (nodes[:, 0] == ref.N).all() and (nodes[:, 3] == ref.VL).all()
    assert (nodes[:, 4] == ref.child_begin).all() and (nodes[:, 5] == ref.child_count).all()
    assert (nodes[:, 6] == ref.action).all()
    assert np.allclose(nodes[:, 2], ref.P, rtol=0, atol=1e-8)           # printed with 9 digits: exact to the float
    assert np.abs(nodes[:, 1] - ref.W).max() <= 1e-5 * max(1.0, np.abs(ref.W).max())
    assert ref.N[0] == sims                                            # every simulation backed up through the root
    want, children = ref.action_probabilities(0, 0.0, CELLS)
    assert children == ref.child_count[0] and (probs == want).all()
    assert int(head[1]) == int(np.argmax(want))                        # temperature 0: the most visited move
    assert abs(float(head[3]) - float(ref.W[0]) / sims) < 1e-5
    if widening:
        assert ref.child_count[0] == 8                                 # root expanded at N = 0: max(8, 2 * 1) of 11 moves
        assert ref.child_count[ref.child_count > 0].max() <= 11
        # the children kept are a random subset of the legal moves, not the moves of lowest index at every node
        kept = [tuple(sorted(nodes[int(b):int(b + c), 6].astype(int))) for b, c in zip(nodes[:, 4], nodes[:, 5]) if c == 8]
        assert any(k != tuple(range(k[0], k[0] + 8)) and k[-1] > 8 for k in kept)
        assert len({k for k in kept}) > 1
    else:
        assert ref.child_count[0] == 11
    # a terminal state is answered without a search: the side to move has lost
    assert lines[-1] == "terminal action -1 value -1 probabilities 12"


@pytest.mark.gpu
@pytest.mark.parametrize("widening", [0, 1])
def test_search_that_follows_transpositions_matches_the_checker(widening):
    """settings.follow_transpositions: every batch is selected by the loop that stores, looks up and REDIRECTS
    (reference mcts_engine_batch_tree_simple.cpp:88-165), every new child keyed by the game's own hash when it
    is created; the mock game's key does not depend on the order of the moves, so transpositions abound.  The
    whole search replayed through the checker: every node, the redirects counted, the move probabilities."""
    sims, batch = 300, 16
    r = subprocess.run([EXE, "search", str(sims), str(batch), str(widening), "0", "0", "1", "1"], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().split("\n")
    head = lines[0].split()
    probs = np.array([float(x) for x in next(ln for ln in lines if ln.startswith("probabilities")).split()[1:]], np.float32)
    table = next(ln for ln in lines if ln.startswith("table entries")).split()
    nodes = np.array([[float(x) for x in ln.split()[2:]] for ln in lines if ln.startswith("node ")])
    ref = replay_search(sims, batch, widening, follow=True)
    assert (int(table[2]), int(table[4])) == ref.table_counts, (table, ref.table_counts)
    assert ref.table_counts[1] > 0 and (ref.alias >= 0).any()          # slots were re-pointed
    assert int(head[7]) == ref.n == len(nodes)
    assert (nodes[:, 0] == ref.N).all() and (nodes[:, 3] == ref.VL).all()
    assert (nodes[:, 4] == ref.child_begin).all() and (nodes[:, 5] == ref.child_count).all()
    assert (nodes[:, 6] == ref.action).all()
    assert np.abs(nodes[:, 1] - ref.W).max() <= 1e-5 * max(1.0, np.abs(ref.W).max())
    assert ref.N[0] == sims
    # the probabilities count the visits of the nodes the root's slots hold
    held = np.where(ref.alias >= 0, ref.alias, np.arange(ref.n)).astype(np.int32)
    seen = R.RefTree(N=ref.N[held], W=ref.W, P=ref.P, VL=ref.VL, child_begin=ref.child_begin, child_count=ref.child_count,
                     action=ref.action)
    want, children = seen.action_probabilities(0, 0.0, CELLS)
    assert children == ref.child_count[0] and (probs == want).all()


@pytest.mark.gpu
def test_second_search_on_one_engine_starts_from_an_empty_table():
    """Node ids start again at 0 with every search's new tree; entries of the table that point into the old
    tree must not be found (the reference's entries are weak pointers that die with it)."""
    sims, batch = 150, 16
    r = subprocess.run([EXE, "search", str(sims), str(batch), "1", "0", "0", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().split("\n")
    table = next(ln for ln in lines if ln.startswith("table entries")).split()
    nodes = np.array([[float(x) for x in ln.split()[2:]] for ln in lines if ln.startswith("node ")])
    ref = replay_search(sims, batch, 1, searches=2)
    assert (int(table[2]), int(table[4])) == ref.table_counts, (table, ref.table_counts)
    assert len(nodes) == ref.n and (nodes[:, 0] == ref.N).all() and (nodes[:, 6] == ref.action).all()


@pytest.mark.gpu
def test_search_with_noise_and_temperature_runs_and_is_consistent():
    r = subprocess.run([EXE, "search", "200", "16", "1", "1", "1.0"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().split("\n")
    head = lines[0].split()
    probs = np.array([float(x) for x in next(ln for ln in lines if ln.startswith("probabilities")).split()[1:]])
    nodes = np.array([[float(x) for x in ln.split()[2:]] for ln in lines if ln.startswith("node ")])
    assert abs(probs.sum() - 1.0) < 1e-4 and probs[int(head[1])] > 0   # the move was drawn from the distribution
    kids = nodes[int(nodes[0, 4]):int(nodes[0, 4] + nodes[0, 5])]
    assert nodes[0, 0] == 200 and kids[:, 0].sum() == 199              # the root's own evaluation is the first simulation
    assert abs(kids[:, 2].sum() - 1.0) < 0.35 and (kids[:, 2] > 0).all()   # priors mixed with noise, still a rough distribution
    assert (probs[kids[:, 6].astype(int)] > 0).sum() == (kids[:, 0] > 0).sum()


@pytest.mark.gpu
def test_flatten_tree_lays_a_pointer_tree_out_breadth_first_and_searches_on():
    r = subprocess.run([EXE, "flatten"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    flat = np.array([[float(x) for x in ln.split()[2:]] for ln in r.stdout.split("\n") if ln.startswith("flat ")])
    # root, its three children in vector order, then the grandchildren in the same order
    assert flat[:, 0].tolist() == [40, 20, 12, 7, 9, 10, 6]
    assert flat[:, 6].tolist() == [1, 4, 0, 6, 0, 0, 0] and flat[:, 7].tolist() == [3, 2, 0, 1, 0, 0, 0]
    assert flat[:, 8].tolist() == [-1, 7, 2, 9, 1, 4, 5]
    assert flat[:, 1].tolist() == [4.0, 8.0, -3.0, 0.5, 2.25, -5.0, 1.5]        # value sums back from the means
    # a node type with accessors of the stored sums: taken as they are, where mean * visits would lose the last bit
    sums = next(ln for ln in r.stdout.split("\n") if ln.startswith("sums exact")).replace(",", "").split()
    assert int(sums[2]) == int(sums[4]) == 40 and int(sums[-1]) > 0, sums
    assert flat[:, 3].tolist() == [0, 0, 3, 0, 0, 0, 0] and flat[:, 4].tolist() == [0, 10, 6, 3, 4, 5, 3]
    ref = R.RefTree(N=flat[:, 0], W=flat[:, 1], P=flat[:, 2], VL=flat[:, 3], child_begin=flat[:, 6], child_count=flat[:, 7],
                    action=flat[:, 8])
    paths, plen, leaf, _ = ref.select_batch(np.zeros(6, np.int32), R.make_params(c_puct=1.4, virtual_loss=3, max_depth=4))
    acts = ref.gather_actions(paths, plen)
    got = [ln for ln in r.stdout.split("\n") if ln.startswith("path")]
    for t, ln in enumerate(got):
        ids = [int(x) for x in ln.split(" moves")[0].split()[1:]]
        mv = [int(x) for x in ln.split(" moves")[1].split()]
        assert ids == paths[t, :plen[t]].tolist() and mv == acts[t, :plen[t] - 1].tolist()


def test_search_driver_reports_errors_without_a_gpu():
    assert os.path.exists(EXE), "build the adapter first (python -m omoknuni_small_amd.build)"
    r = subprocess.run([EXE, "flatten"], capture_output=True, text=True, timeout=120)
    if r.returncode == 1:
        assert "omk_forest_create" in r.stderr          # no device: an exception with the library's message, no crash
    else:
        assert r.returncode == 0
