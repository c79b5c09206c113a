"""The checker's leaf expansion against what the reference fixes about MCTSNode::expand and
setPriorProbabilities: its own unit tests (tests/mcts/mcts_node_test.cpp:124-170: children =
legal moves, the node stops being a leaf, actions in range; :175-200: a terminal state is not
expanded) and the rules read off src/mcts/mcts_node.cpp:238-436, :512-593 (uniform prior of
expand, clamp to [0,1], 0.01 for a move outside the action space, first caller wins, 1000-move
limit).  The order of the children is random in the reference; the checker keeps the order
given, which is one of its outcomes."""
import numpy as np

from oracle import ref_cpu as R


def leaf_tree(n=1):
    z = np.zeros(n, np.int32)
    return R.RefTree(N=z + 5, W=np.zeros(n, np.float32), P=np.ones(n, np.float32), VL=z, child_begin=z, child_count=z,
                     action=z - 1)


def test_three_legal_moves_give_three_children():
    t = leaf_tree()
    first = t.expand_batch([0], [0, 3], [2, 0, 1])
    assert first.tolist() == [1] and t.n == 4
    assert t.child_begin[0] == 1 and t.child_count[0] == 3          # not a leaf any more
    assert t.action[1:4].tolist() == [2, 0, 1]                      # one child per move, each in range
    assert (t.N[1:4] == 0).all() and (t.W[1:4] == 0).all() and (t.VL[1:4] == 0).all()
    assert (t.child_count[1:4] == 0).all()                          # children are leaves
    assert np.allclose(t.P[1:4], np.float32(1.0) / np.float32(3.0), rtol=0, atol=0)
    assert t.N[0] == 5                                              # the node's own statistics are untouched


def test_terminal_state_is_not_expanded():
    t = leaf_tree()
    first = t.expand_batch([0], [0, 0], [])
    assert first.tolist() == [-1] and t.n == 1 and t.child_count[0] == 0


def test_priors_follow_the_policy_with_clamp_and_default():
    t = leaf_tree()
    policy = np.array([[-0.2, 0.25, 1.7, 0.5]], np.float32)
    t.expand_batch([0], [0, 5], [0, 1, 2, 3, 9], policy=policy, action_space=4)
    assert t.P[1:6].tolist() == [0.0, 0.25, 1.0, 0.5, np.float32(0.01)]


def test_first_traversal_wins_a_shared_leaf_and_ids_follow_traversal_order():
    t = leaf_tree(3)
    # traversals: 0 -> leaf 2, 1 -> leaf 1 (terminal), 2 -> leaf 2 again, 3 -> leaf 0
    first = t.expand_batch([2, 1, 2, 0], [0, 2, 2, 5, 6], [7, 8, 1, 2, 3, 4])
    assert first.tolist() == [3, -1, -1, 5]
    assert (t.child_begin[2], t.child_count[2]) == (3, 2) and t.action[3:5].tolist() == [7, 8]
    assert t.child_count[1] == 0
    assert (t.child_begin[0], t.child_count[0]) == (5, 1) and t.action[5] == 4
    assert t.n == 6


def test_expanded_node_is_left_alone():
    t = leaf_tree()
    t.expand_batch([0], [0, 2], [0, 1])
    before = (t.child_begin.copy(), t.child_count.copy(), t.P.copy())
    first = t.expand_batch([0], [0, 3], [5, 6, 7])
    assert first.tolist() == [-1] and t.n == 3
    assert (t.child_begin == before[0]).all() and (t.child_count == before[1]).all() and (t.P == before[2]).all()


def test_move_list_is_cut_at_the_reference_limit():
    t = leaf_tree()
    t.expand_batch([0], [0, 1500], np.arange(1500))
    assert t.child_count[0] == 1000 and t.n == 1001 and t.action[1000] == 999


def test_widening_child_count_closed_forms():
    """mcts_node.cpp:305-308: min(legal, size_t(max(8.0f, float(cpw * pow(N + 1, kpw))))), at least one
    child; off = every legal move.  The reference's own test only fixes >= 4 and <= legal
    (tests/mcts/progressive_widening_test.cpp:124-139)."""
    W = R.lib().ref_widened_children
    assert W(30, 0, 0, 2.0, 0.5) == 30                      # widening off: all legal moves
    assert W(30, 0, 1, 2.0, 0.5) == 8                       # 2 * 1^0.5 = 2 -> the floor of 8
    assert W(5, 0, 1, 2.0, 0.5) == 5                        # fewer legal moves than the floor
    assert W(30, 15, 1, 2.0, 0.5) == 8                      # 2 * sqrt(16) = 8
    assert W(30, 24, 1, 2.0, 0.5) == 10                     # 2 * sqrt(25) = 10
    assert W(30, 35, 1, 2.0, 0.5) == 12                     # 2 * 6
    assert W(30, 3, 1, 2.0, 1.0) == 8 and W(30, 4, 1, 2.0, 1.0) == 10      # k = 1: 2 * (N + 1)
    assert W(30, 10 ** 6, 1, 2.0, 0.5) == 30                # never more than the legal moves
    assert W(400, 2 ** 31 - 2, 1, 1e30, 3.0) == 400         # a target beyond any integer: all of them
    assert W(1, 0, 1, 2.0, 0.5) == 1
    # the truncation toward zero of the float: 2 * sqrt(20) = 8.94 -> 8, 2 * sqrt(21) = 9.17 -> 9
    assert W(30, 19, 1, 2.0, 0.5) == 8 and W(30, 20, 1, 2.0, 0.5) == 9
    for n in range(0, 3000, 7):                             # against the formula in Python doubles / float32
        want = min(50, int(max(np.float32(8.0), np.float32(2.0 * float(n + 1) ** 0.5))))
        assert W(50, n, 1, 2.0, 0.5) == want
        assert 4 <= W(50, n, 1, 2.0, 0.5) <= 50             # the reference-test fact


def test_widening_keeps_the_first_moves_offered_and_their_uniform_prior():
    t = leaf_tree(2)
    t.N[:] = [24, 0]
    first = t.expand_batch([0, 1], [0, 20, 40], np.arange(40) % 20, widening=(2.0, 0.5))
    assert first.tolist() == [2, 12]
    assert (t.child_begin[0], t.child_count[0]) == (2, 10) and t.action[2:12].tolist() == list(range(10))
    assert (t.child_begin[1], t.child_count[1]) == (12, 8) and t.action[12:20].tolist() == list(range(8))
    assert (t.P[2:12] == np.float32(1.0) / np.float32(10.0)).all()      # 1 / children, not 1 / legal moves
    assert (t.P[12:20] == np.float32(1.0) / np.float32(8.0)).all()
    assert t.n == 20
    # an expanded node is left alone, however many visits it has by now (the incremental branch of
    # expand() sits behind a compare-exchange that returns first)
    t.N[0] = 10 ** 6
    assert t.expand_batch([0], [0, 20], np.arange(20), widening=(2.0, 0.5)).tolist() == [-1] and t.n == 20


def test_policy_branches_of_set_prior_probabilities():
    """:537-560 a policy over the action space, :561-575 one value per child, :576-584 any other length
    -> uniform; an empty policy means setPriorProbabilities is not called at all."""
    t = leaf_tree(4)
    A = 6
    pol = np.array([0.5, 0.1, 0.2, 0.05, 0.1, 0.05,       # traversal 0: the action space
                    0.7, -0.3, 1.5,                        # traversal 1: as many as children (3), clamped
                    0.2, 0.8,                              # traversal 2: neither (4 children, 2 values)
                    ], np.float32)                         # traversal 3: empty
    pb = [0, 6, 9, 11, 11]
    t.expand_batch([0, 1, 2, 3], [0, 3, 6, 10, 12], [4, 0, 9, 1, 2, 3, 0, 1, 2, 3, 5, 4], policy=pol, action_space=A,
                   policy_begin=pb)
    assert t.P[4:7].tolist() == [np.float32(0.1), 0.5, np.float32(0.01)]           # by action; 9 is outside
    assert t.P[7:10].tolist() == [np.float32(0.7), 0.0, 1.0]                       # by child index, clamped
    assert (t.P[10:14] == np.float32(0.25)).all()                                  # mismatch: uniform
    assert (t.P[14:16] == np.float32(0.5)).all()                                   # no policy: expand's uniform
    # when the action space has as many entries as the node has children, the action branch wins
    t2 = leaf_tree()
    t2.expand_batch([0], [0, 3], [2, 0, 1], policy=np.array([0.1, 0.2, 0.7], np.float32), action_space=3, policy_begin=[0, 3])
    assert t2.P[1:4].tolist() == [np.float32(0.7), np.float32(0.1), np.float32(0.2)]


def test_selection_descends_into_new_children():
    t = leaf_tree()
    t.expand_batch([0], [0, 3], [0, 1, 2], policy=np.array([[0.1, 0.7, 0.2]], np.float32), action_space=3)
    p = R.make_params(c_puct=1.4, virtual_loss=3, max_depth=4)
    paths, plen, leaf, _ = t.select_batch(np.zeros(2, np.int32), p)
    assert plen.tolist() == [2, 2]
    assert leaf[0] == 2           # all children unvisited: the largest prior wins (sqrt(N_parent) > 0)


# ---- MCTSEngine::getActionProbabilities (src/mcts/mcts_engine_tree.cpp:388-465) ----

def counts_tree(counts, actions=None):
    k = len(counts)
    z = np.zeros(k + 1, np.int32)
    cb, cc = z.copy(), z.copy()
    cb[0], cc[0] = 1, k
    act = np.concatenate([[-1], np.arange(k) if actions is None else actions]).astype(np.int32)
    return R.RefTree(N=np.concatenate([[sum(counts)], counts]).astype(np.int32), W=np.zeros(k + 1, np.float32),
                     P=np.ones(k + 1, np.float32), VL=z, child_begin=cb, child_count=cc, action=act)


def test_probabilities_near_zero_temperature_pick_the_first_maximum():
    p, n = counts_tree([3, 9, 9, 1]).action_probabilities(0, 0.001, 6)
    assert n == 4 and p.tolist() == [0, 1, 0, 0, 0, 0]


def test_probabilities_at_temperature_one_are_proportional_to_visits():
    p, _ = counts_tree([1, 2, 5, 0]).action_probabilities(0, 1.0, 4)
    # (count/max)^(1/1) normalised in binary32, in child order
    s = np.float32(0)
    scaled = [np.float32(np.float32(c) / np.float32(5)) for c in (1, 2, 5)]
    for x in scaled:
        s = np.float32(s + x)
    assert p.tolist() == [np.float32(x / s) for x in scaled] + [0.0]
    assert abs(float(p.sum()) - 1.0) < 1e-6


def test_probabilities_sharpen_with_low_temperature():
    p, _ = counts_tree([2, 4]).action_probabilities(0, 0.5, 2)
    assert np.allclose(p, [0.2, 0.8], rtol=1e-6)      # (1/2)^2 : 1


def test_probabilities_uniform_when_nothing_was_visited_and_empty_without_children():
    p, n = counts_tree([0, 0, 0, 0]).action_probabilities(0, 1.0, 5)
    assert n == 4 and p.tolist() == [0.25, 0.25, 0.25, 0.25, 0.0]
    t = counts_tree([1, 2])
    p, n = t.action_probabilities(1, 1.0, 3)          # a leaf
    assert n == 0 and p.tolist() == [0.0, 0.0, 0.0]


def test_probabilities_are_laid_out_by_action_and_skip_actions_outside_the_space():
    p, _ = counts_tree([1, 1, 2], actions=[4, 9, 0]).action_probabilities(0, 1.0, 6)
    assert p[4] == 0.25 and p[0] == 0.5 and p.sum() == 0.75   # action 9 is outside: dropped


# ---- tree reuse (src/mcts/mcts_engine_search.cpp:1029-1075) ----

def test_reroot_picks_the_first_child_with_the_action():
    t = counts_tree([1, 2, 3, 4], actions=[7, 5, 7, 2])
    assert t.reroot_child(0, 7) == 1          # children in order: the first match
    assert t.reroot_child(0, 2) == 4
    assert t.reroot_child(0, 9) == -1         # no such child: the reference starts afresh
    assert t.reroot_child(0, -1) == -1        # last_action < 0: no reuse
    assert t.reroot_child(1, 7) == -1         # a leaf has no children


def test_compaction_keeps_the_subtree_in_breadth_first_sibling_order():
    from tests.helpers import random_tree
    soa, roots = random_tree(5, n_expand=30, fanout=(2, 6), max_depth=4)
    t = R.RefTree.from_soa(soa)
    kid = int(soa["child_begin"][roots[0]]) + 1
    t2, order = t.compacted(kid)
    assert order[0] == kid and len(set(order.tolist())) == len(order)
    # every kept node keeps its statistics, and children stay contiguous in the old order
    assert (t2.N == t.N[order]).all() and (t2.child_count == t.child_count[order]).all()
    for i in range(t2.n):
        for j in range(t2.child_count[i]):
            assert order[t2.child_begin[i] + j] == t.child_begin[order[i]] + j
    # exactly the descendants of the new root were kept
    keep, stack = set(), [kid]
    while stack:
        x = stack.pop()
        keep.add(x)
        stack.extend(range(t.child_begin[x], t.child_begin[x] + t.child_count[x]))
    assert keep == set(order.tolist())
    # the same selections, node for node, before and after
    p = R.make_params(c_puct=1.4, virtual_loss=3, max_depth=6)
    pa, la, _, _ = R.RefTree.from_soa(soa).select_batch(np.full(40, kid, np.int32), p)
    pb, lb, _, _ = t2.select_batch(np.zeros(40, np.int32), p)
    assert (la == lb).all()
    for i in range(40):
        assert (order[pb[i, :lb[i]]] == pa[i, :la[i]]).all()


# ---- RAVE statistics of backPropagate (src/mcts/mcts_engine_tree.cpp:288-331) ----

def test_rave_backup_updates_children_whose_action_is_on_the_path():
    # root(0) -> children 1,2,3 with actions 5,6,7; node 1 -> children 4,5 with actions 6,9
    z = lambda *v: np.array(v, np.int32)
    t = R.RefTree(N=z(3, 1, 1, 1, 0, 0), W=np.zeros(6, np.float32), P=np.ones(6, np.float32), VL=z(0, 0, 0, 0, 0, 0),
                  child_begin=z(1, 4, 0, 0, 0, 0), child_count=z(3, 2, 0, 0, 0, 0), action=z(-1, 5, 6, 7, 6, 9),
                  rN=np.zeros(6, np.int32), rW=np.zeros(6, np.float32))
    # one path root -> 1 -> 4: its actions are {5, 6} (the root's -1 does not count)
    t.rave_backup_batch(np.array([[0, 1, 4]], np.int32), [3], [0.5])
    # at the leaf (4): no children.  at node 1 (sign flipped once): child 4 (action 6) matches, child 5 does not.
    # at the root (flipped twice): children 1 (action 5) and 2 (action 6) match, child 3 does not.
    assert t.rN.tolist() == [0, 1, 1, 0, 1, 0]
    assert t.rW.tolist() == [0.0, 0.5, 0.5, 0.0, -0.5, 0.0]


# ---- Dirichlet noise on the root priors (src/mcts/mcts_engine_eval.cpp:78-110) ----

def test_root_noise_mixes_normalised_samples_into_the_priors():
    z = lambda *v: np.array(v, np.int32)
    t = R.RefTree(N=z(1, 0, 0, 0, 0), W=np.zeros(5, np.float32), P=np.array([0, .5, .25, .125, .125], np.float32),
                  VL=z(0, 0, 0, 0, 0), child_begin=z(1, 0, 0, 0, 0), child_count=z(4, 0, 0, 0, 0))
    assert t.add_root_noise(0, [1.0, 3.0, 0.0, 4.0], 0.25) == 4
    # noise = samples / 8 = .125 .375 0 .5 ; prior = .75 * prior + .25 * noise  (all exact in binary32)
    assert t.P.tolist() == [0.0, 0.40625, 0.28125, 0.09375, 0.21875]
    assert abs(float(t.P[1:].sum()) - 1.0) < 1e-6   # a distribution stays one
    # samples that sum to zero: uniform noise (:98-101)
    t.add_root_noise(0, [0.0, 0.0, 0.0, 0.0], 0.5)
    assert t.P.tolist() == [0.0, 0.328125, 0.265625, 0.171875, 0.234375]
    # a root without children is left alone (:78-80)
    assert t.add_root_noise(2, [], 0.25) == 0
