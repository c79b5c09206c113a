"""Position keys of the checker: the std::mt19937_64 stream of utils::ZobristHash
(reference src/utils/zobrist_hash.cpp:9-36,129-131), GomokuState::compute_hash_signature_internal
(src/games/gomoku/gomoku_state.cpp:947-957) and the replayed state of the traversal loop
(src/mcts/mcts_engine_batch_tree_simple.cpp:119-124,133-137).

Pinned by: the known answers of the generator the C++ standard fixes (first output and the
10000th of a default-seeded std::mt19937_64), the structure of the constructor's loops, and the
algebra of the key (XOR of piece keys and side key: order of moves irrelevant, a stone folded in
twice cancels, a single stone changes the key by exactly its piece key and the side swap)."""
import numpy as np
import pytest

from oracle import ref_cpu as R
from tests.helpers import board_forest


def test_mt19937_64_known_answers():
    out = R.mt19937_64(5489, 10000)
    assert int(out[0]) == 14514284786278117030           # first output of the default seed
    assert int(out[9999]) == 9981545732273789042         # [rand.predef]: 10000th invocation


def test_table_order_of_the_constructor():
    bs = 9
    piece, player = R.zobrist_tables(bs, 2, 4, 1234)
    stream = R.mt19937_64(1234, 2 * bs * bs + 4)
    assert (piece[0] == stream[:bs * bs]).all()          # piece type 0 first, positions ascending
    assert (piece[1] == stream[bs * bs:2 * bs * bs]).all()
    assert (player == stream[2 * bs * bs:]).all()        # player keys after all piece tables
    with pytest.raises(ValueError):
        R.zobrist_tables(bs, 2, 4, 0)                    # seed 0 = clock in the reference
    with pytest.raises(ValueError):
        R.zobrist_tables(0, 2, 4, 1)


def test_position_key_algebra():
    cells = 225
    rng = np.random.default_rng(5)
    piece = rng.integers(0, 2**63, (2, cells), dtype=np.uint64)
    player = rng.integers(0, 2**63, 2, dtype=np.uint64)
    empty = np.zeros(cells, np.int8)
    assert R.position_key(empty, piece, player, 1) == int(player[0])
    assert R.position_key(empty, piece, player, 2) == int(player[1])
    b = empty.copy()
    b[17] = 1
    assert R.position_key(b, piece, player, 2) == int(piece[0, 17] ^ player[1])
    b[200] = 2
    assert R.position_key(b, piece, player, 1) == int(piece[0, 17] ^ piece[1, 200] ^ player[0])
    # a full random board: the XOR of what is on it, whatever the order
    b = rng.integers(0, 3, cells).astype(np.int8)
    want = int(player[0])
    for c in rng.permutation(cells):
        if b[c]:
            want ^= int(piece[b[c] - 1, c])
    assert R.position_key(b, piece, player, 1) == want


def test_replayed_paths_against_the_closed_form():
    """The key of a replayed path equals root key ^ piece keys of its moves (mover alternating from the
    root's side to move) ^ the two side keys when the number of moves is odd; transposed move orders
    meet in one key."""
    cells = 81
    soa, roots, boards, players = board_forest(11, cells=cells, root_stones=12, n_expand=60, fanout=(2, 9),
                                               max_depth=6, n_roots=3)
    tree = R.RefTree.from_soa(soa)
    rng = np.random.default_rng(2)
    piece = rng.integers(0, 2**63, (2, cells), dtype=np.uint64)
    player = rng.integers(0, 2**63, 2, dtype=np.uint64)
    B = 48
    troots = np.repeat(roots, B // len(roots)).astype(np.int32)
    rp = R.make_params(c_puct=1.4, virtual_loss=3, max_depth=6)
    paths, plen, leaf, _ = tree.select_batch(troots, rp)
    ri = np.repeat(np.arange(len(roots)), B // len(roots))
    keys, bad = R.leaf_keys(tree, paths, plen, boards[ri], players[ri], piece, player)
    assert bad == 0
    assert plen.max() >= 3
    for t in range(B):
        p0 = int(players[ri[t]]) - 1
        h = R.position_key(boards[ri[t]], piece, player, p0 + 1)
        for d in range(1, plen[t]):
            h ^= int(piece[(p0 + d - 1) & 1, soa["action"][paths[t, d]]])
        if (plen[t] - 1) & 1:
            h ^= int(player[0] ^ player[1])
        assert h == int(keys[t]), t
    # same stones, other order: one key (what the transposition table relies on)
    b = np.zeros(cells, np.int8)
    b[3], b[40], b[7] = 1, 2, 1
    k1 = R.position_key(b, piece, player, 2)
    assert k1 == int(piece[0, 7] ^ piece[1, 40] ^ piece[0, 3] ^ player[1])


def test_bad_paths_are_reported():
    cells = 25
    soa, roots, boards, players = board_forest(3, cells=cells, root_stones=4, n_expand=6, fanout=(2, 4), max_depth=3)
    tree = R.RefTree.from_soa(soa)
    rng = np.random.default_rng(1)
    piece = rng.integers(0, 2**63, (2, cells), dtype=np.uint64)
    player = rng.integers(0, 2**63, 2, dtype=np.uint64)
    rp = R.make_params(max_depth=3)
    paths, plen, _, _ = tree.select_batch(np.array([roots[0]] * 2, np.int32), rp)
    occupied = boards.copy()
    occupied[0, soa["action"][paths[0, 1]]] = 1          # the first move lands on a stone
    keys, bad = R.leaf_keys(tree, paths, plen, np.repeat(occupied, 2, 0), np.repeat(players, 2), piece, player)
    assert bad >= 1 and int(keys[0]) == 2**64 - 1
