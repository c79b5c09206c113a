"""The checker's traversal loop with the transposition table on (ref_select_redirect_batch: flat arrays, an
alias per child slot) against a LITERAL restatement of the reference's loop
(src/mcts/mcts_engine_batch_tree_simple.cpp:88-165: select, virtual loss, record the move, store the
unvisited child, look the position up, and on a transposition revert / updateChildReference / apply,
:142-156; MCTSNode::updateChildReference src/mcts/mcts_node.cpp:617-630) over node OBJECTS whose
children are Python lists that the redirect re-points, with the game's own getHash() of the replayed
move list as the key and the dict-based table of test_oracle_tt as the table.

Games: the reference's own collision fixture (tests/mcts/transposition_table_test.cpp:15-232: two
moves per position, four plies, getHash() equal for the move lists that start [0, 1] and [1, 0]) and a
small stone-placing game whose key does not depend on the order of a side's stones.  The per-child
scores themselves come from the checker (they are pinned by the known-answer table elsewhere); what
is pinned here is the loop: which node a slot holds, where virtual loss goes, what is stored and
found when, the recorded moves, the paths."""
import numpy as np
import pytest

from oracle import ref_cpu as R
from tests.test_oracle_tt import DictTable, same_content

M64 = (1 << 64) - 1


def fixture_hash(moves, create_transpositions=True):
    """TranspositionGameState::getHash (transposition_table_test.cpp:94-128) of a move history."""
    depth = len(moves)
    player = 1 if depth % 2 == 0 else 2
    h = 0
    h = (h * 31 + depth) & M64
    h = (h * 31 + player) & M64
    if create_transpositions and len(moves) >= 2 and sorted(moves[:2]) == [0, 1]:
        h = (h * 31 + 42) & M64
        rest = moves[2:]
    else:
        rest = moves
    for m in rest:
        h = (h * 31 + m) & M64
    return h


def fixture_tree(rng, plies=4):
    """The fixture's game tree, fully expanded: ids breadth-first, children of a node contiguous."""
    hist = [[]]
    cb, cc, action = [], [], [-1]
    i = 0
    while i < len(hist):
        if len(hist[i]) < plies:
            cb.append(len(hist))
            cc.append(2)
            for m in (0, 1):
                hist.append(hist[i] + [m])
                action.append(m)
        else:
            cb.append(0)
            cc.append(0)
        i += 1
    n = len(hist)
    P = rng.uniform(0.2, 0.8, n).astype(np.float32)
    keys = np.array([fixture_hash(h) for h in hist], np.uint64)
    return dict(n=n, cb=np.array(cb, np.int32), cc=np.array(cc, np.int32), action=np.array(action, np.int32), P=P,
                keys=keys, hist=hist, game_hash=lambda mv: fixture_hash(list(mv)))


def stones_tree(rng, cells=5, plies=4):
    """A stone-placing game (a cell is played once, sides alternate), fully expanded to `plies`; the key of a
    position is a function of the two sides' stone SETS, so move orders that place the same stones transpose."""
    salt = rng.integers(1, 1 << 62, (2, cells), dtype=np.uint64)

    def key(moves):
        if len(set(moves)) != len(moves) or len(moves) > plies or any(m < 0 or m >= cells for m in moves):
            return None          # no such position in the game (the reference's makeMove would throw)
        h = np.uint64(len(moves) * 0x9E3779B97F4A7C15 & M64)
        for ply, m in enumerate(moves):
            h ^= salt[ply & 1, m]
        return int(h)

    hist = [[]]
    cb, cc, action = [], [], [-1]
    i = 0
    while i < len(hist):
        free = [m for m in range(cells) if m not in hist[i]]
        if len(hist[i]) < plies and free:
            cb.append(len(hist))
            cc.append(len(free))
            for m in free:
                hist.append(hist[i] + [m])
                action.append(m)
        else:
            cb.append(0)
            cc.append(0)
        i += 1
    n = len(hist)
    P = rng.uniform(0.05, 0.9, n).astype(np.float32)
    keys = np.array([key(h) for h in hist], np.uint64)
    return dict(n=n, cb=np.array(cb, np.int32), cc=np.array(cc, np.int32), action=np.array(action, np.int32), P=P,
                keys=keys, hist=hist, game_hash=key)


class Node:
    def __init__(self, nid, action):
        self.id = nid
        self.action = action
        self.children = []


def object_tree(g):
    nodes = [Node(i, int(g["action"][i])) for i in range(g["n"])]
    for i in range(g["n"]):
        nodes[i].children = [nodes[g["cb"][i] + c] for c in range(g["cc"][i])]
    return nodes


def literal_select_child(tree, node, params):
    """MCTSNode::selectChild (mcts_node.cpp:90-236) over node.children: first scan, strict >, then the
    second scan with the best score carried over; the fallback to the least visited child."""
    best, best_score = None, -np.inf
    for ch in node.children:
        s1, _ = tree.child_scores(node.id, ch.id, params)
        if s1 > best_score:
            best, best_score = ch, s1
    if best is None:
        if node.children:
            lo = None
            for ch in node.children:
                if lo is None or tree.N[ch.id] < lo:
                    lo, best = tree.N[ch.id], ch
        return best
    for ch in node.children:
        _, s2 = tree.child_scores(node.id, ch.id, params)
        if s2 > best_score:
            best, best_score = ch, s2
    return best


def literal_batch(tree, nodes, root, B, params, table, clock, game_hash):
    """mcts_engine_batch_tree_simple.cpp:88-165 for B traversals, one after the other.  The table's access
    counter starts at `clock` and ticks where the reference's does: on a store that finds its key
    (phmap_transposition_table.cpp:65) and on a lookup that returns an entry (:107).  Returns the counter
    as its last element."""
    vl = params.virtual_loss
    out_paths, out_moves, redirects, g = [], [], 0, 0
    for _ in range(B):
        current = nodes[root]
        path, moves = [current.id], []
        while current.children and len(path) <= params.max_depth:
            best = literal_select_child(tree, current, params)
            if best is None:
                break
            tree.add_vl(best.id, vl)                                   # :109
            moves.append(best.action)                                  # :112
            h = game_hash(moves)                                       # :119-124, :133-137
            if h is not None:
                if tree.N[best.id] == 0:                               # :116
                    if table.store(tree, h, best.id, len(moves), clock) != "new":
                        clock += 1
                tt = table.lookup(h, 0, clock)                         # :141
                if tt >= 0:
                    clock += 1
                if tt >= 0 and tt != best.id and tree.N[tt] > 0:       # :142
                    tree.remove_vl(best.id, vl)                        # :146
                    idx = [c is best for c in current.children].index(True)   # updateChildReference: first match
                    current.children[idx] = nodes[tt]
                    tree.add_vl(tt, vl)                                # :152
                    best = nodes[tt]
                    redirects += 1
            g += 1
            current = best
            path.append(current.id)
        out_paths.append(path)
        out_moves.append(moves)
    return out_paths, out_moves, redirects, g, clock


def run_search(g, seed, batches, B, vl=3, c_puct=1.4, max_depth=8):
    rng = np.random.default_rng(seed)
    n = g["n"]
    z = np.zeros(n, np.int32)
    mk = lambda: R.RefTree(N=z, W=np.zeros(n, np.float32), P=g["P"], VL=z, child_begin=g["cb"], child_count=g["cc"],
                           action=g["action"])
    flat, lit = mk(), mk()
    nodes = object_tree(g)
    alias = np.full(n, -1, np.int32)
    tt, table = R.RefTT(10), DictTable()
    params = R.make_params(c_puct=c_puct, virtual_loss=vl, max_depth=max_depth)
    total_redirects = 0
    for _ in range(batches):
        t0 = tt.clock
        paths, plen, leaf, moves, counts = flat.select_redirect_batch(np.zeros(B, np.int32), params, tt, g["keys"], alias)
        lp, lm, lr, lg, lclock = literal_batch(lit, nodes, 0, B, params, table, t0, g["game_hash"])
        assert counts[4] == lg and tt.clock == lclock
        for i in range(B):
            assert paths[i, :plen[i]].tolist() == lp[i], (i, paths[i], lp[i])
            assert (paths[i, plen[i]:] == -1).all() and leaf[i] == lp[i][-1]
            assert moves[i, :plen[i] - 1].tolist() == lm[i]
        assert counts[3] == lr
        total_redirects += lr
        # every slot holds the node the objects' children lists hold
        for i in range(n):
            held = [int(alias[s]) if alias[s] >= 0 else int(s) for s in range(g["cb"][i], g["cb"][i] + g["cc"][i])]
            assert held == [c.id for c in nodes[i].children]
        assert (flat.VL == lit.VL).all()
        same_content(tt, table)
        values = rng.uniform(-1, 1, B).astype(np.float32)
        flat.backup_batch(paths, plen, values, vl)
        lit.backup_batch(paths, plen, values, vl)
        assert (flat.N == lit.N).all() and (flat.VL == 0).all()
    return total_redirects, alias, flat


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_collision_fixture_of_the_reference(seed):
    g = fixture_tree(np.random.default_rng(seed))
    redirects, alias, flat = run_search(g, seed, batches=12, B=8)
    assert redirects >= 1
    # the fixture's transposition: the positions [0, 1] and [1, 0] have one key, and one of the two slots
    # has been re-pointed (where to by now is another matter: a re-pointed slot records the action of the
    # node it holds, the replayed position is then another one, and the next lookup re-points it again)
    a, b = g["hist"].index([0, 1]), g["hist"].index([1, 0])
    assert g["keys"][a] == g["keys"][b]
    assert alias[a] >= 0 or alias[b] >= 0


def test_without_transpositions_it_is_the_plain_loop():
    rng = np.random.default_rng(5)
    g = fixture_tree(rng)
    g["keys"] = np.array([fixture_hash(h, False) for h in g["hist"]], np.uint64)
    g["game_hash"] = lambda mv: fixture_hash(list(mv), False)
    redirects, alias, flat = run_search(g, 5, batches=6, B=8)
    assert redirects == 0 and (alias == -1).all()
    # the same search by the loop without a table
    n = g["n"]
    z = np.zeros(n, np.int32)
    plain = R.RefTree(N=z, W=np.zeros(n, np.float32), P=g["P"], VL=z, child_begin=g["cb"], child_count=g["cc"],
                      action=g["action"])
    params = R.make_params(virtual_loss=3, max_depth=8)
    vrng = np.random.default_rng(5)
    for _ in range(6):
        paths, plen, _, _ = plain.select_batch(np.zeros(8, np.int32), params, near_ties=False)
        plain.backup_batch(paths, plen, vrng.uniform(-1, 1, 8).astype(np.float32), 3)
    assert (plain.N == flat.N).all() and (plain.W == flat.W).all()


@pytest.mark.parametrize("seed,vl", [(11, 3), (12, 1), (13, 0)])
def test_stone_game_with_many_transpositions(seed, vl):
    g = stones_tree(np.random.default_rng(seed))
    redirects, alias, _ = run_search(g, seed, batches=25, B=16, vl=vl, max_depth=6)
    assert redirects >= 5
    assert (alias >= 0).sum() >= 3


def test_depth_bound_and_bad_root():
    g = fixture_tree(np.random.default_rng(7))
    redirects, _, _ = run_search(g, 7, batches=10, B=8, max_depth=2)     # paths cut at two steps
    n = g["n"]
    z = np.zeros(n, np.int32)
    t = R.RefTree(N=z, W=np.zeros(n, np.float32), P=g["P"], VL=z, child_begin=g["cb"], child_count=g["cc"])
    with pytest.raises(ValueError):
        t.select_redirect_batch(np.array([n], np.int32), R.make_params(max_depth=4), R.RefTT(6), g["keys"])
