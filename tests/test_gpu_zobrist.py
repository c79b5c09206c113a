"""Position keys of the selected leaves on the device (omk_batch_leaf_keys) against the checker's
replay of reference src/mcts/mcts_engine_batch_tree_simple.cpp:119-124,133-137 + GomokuState::getHash
(src/games/gomoku/gomoku_state.cpp:947-957), through the C ABI.  Bit-exact (64-bit integer work)."""
import numpy as np
import pytest

import omoknuni_small_amd as omk
from omoknuni_small_amd import synth
from oracle import ref_cpu as R
from tests.helpers import board_forest

pytestmark = pytest.mark.gpu


def _tables(cells, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(0, 2**63, (2, cells), dtype=np.uint64), rng.integers(0, 2**63, 2, dtype=np.uint64)


@pytest.mark.parametrize("seed,vl", [(1, 3), (2, 3), (3, 0)])
def test_leaf_keys_match_the_replayed_states(seed, vl):
    cells = 225
    soa, roots, boards, players = board_forest(seed, cells=cells, root_stones=30, n_expand=220, fanout=(2, 14),
                                               max_depth=7, n_roots=4)
    # the tables as the game's own ZobristHash(board_size * board_size, 2, 4, seed) would hold them:
    # the first `cells` keys of each piece table, the first two player keys
    piece_full, player_full = R.zobrist_tables(cells, 2, 4, 99 + seed)
    piece, player = piece_full[:, :cells].copy(), player_full[:2].copy()
    B, D = 256, 7
    ri = np.repeat(np.arange(len(roots)), B // len(roots))
    troots = roots[ri].astype(np.int32)
    tree = R.RefTree.from_soa(soa)
    rp = R.make_params(c_puct=1.4, virtual_loss=vl, max_depth=D)
    rpaths, rlen, rleaf, _ = tree.select_batch(troots, rp)
    want, bad = R.leaf_keys(tree, rpaths, rlen, boards[ri], players[ri], piece, player)
    assert bad == 0
    root_keys = np.array([R.position_key(boards[r], piece, player, players[r]) for r in ri], np.uint64)

    forest = omk.Forest.from_soa(soa)
    batch = omk.Batch(forest, B, D)
    batch.set_roots(troots)
    batch.select(omk.SelectParams(c_puct=1.4, virtual_loss=vl))
    paths, plen, leaf, _ = batch.read()
    assert (paths == rpaths).all() and (plen == rlen).all()
    got = batch.leaf_keys(piece, player, root_keys, players[ri] - 1)
    assert (got == want).all()
    # without virtual loss the visitors of a root all take one path
    assert len(np.unique(got)) > 8 if vl > 0 else len(np.unique(got)) == len(roots)
    assert plen.max() >= (4 if vl > 0 else 2)

    # the keys feed the table: store every leaf under its key, look them up again
    tt = omk.TranspositionTable(forest, 12)
    first = {}
    for t in range(B):
        first.setdefault(int(got[t]), int(leaf[t]))
    tt.insert(got, leaf, plen - 1)
    hit = tt.probe(got)
    assert all(int(hit[t]) == first[int(got[t])] for t in range(B))
    tt.close()
    batch.revert_vl(vl)


def test_leaf_keys_closed_form_at_full_size():
    """256 trees x 50k nodes, one traversal each (the self-play workload): every key is the root key
    with the piece keys of the path's moves folded in, movers alternating, and the side keys
    swapped on an odd number of moves (the synthetic trees do not keep a position, so this is the
    algebra only)."""
    soa, roots, meta = synth.generate("c1", seed=5)
    cells = 225
    piece, player = _tables(cells, 8)
    B, D = meta["n_traversals"], meta["max_depth"]
    troots = synth.traversal_roots(roots, B)
    rng = np.random.default_rng(4)
    root_keys = rng.integers(0, 2**63, B, dtype=np.uint64)
    root_players = rng.integers(0, 2, B).astype(np.int32)
    forest = omk.Forest.from_soa(soa)
    batch = omk.Batch(forest, B, D)
    batch.set_roots(troots)
    batch.select(omk.SelectParams(c_puct=meta["c_puct"], virtual_loss=meta["virtual_loss"]))
    paths, plen, _, actions = batch.read()
    got = batch.leaf_keys(piece, player, root_keys, root_players)
    want = root_keys.copy()
    for d in range(1, D + 1):
        on = plen > d
        side = (root_players + d - 1) & 1
        want[on] ^= piece[side[on], actions[on, d - 1]]
    odd = ((plen - 1) & 1) == 1
    want[odd] ^= player[root_players[odd]] ^ player[root_players[odd] ^ 1]
    assert (got == want).all()
    batch.revert_vl(meta["virtual_loss"])


def test_moves_off_the_board_are_refused():
    soa, roots, boards, players = board_forest(4, cells=225, root_stones=10, n_expand=30, fanout=(2, 8), max_depth=4)
    piece, player = _tables(64, 1)                       # a table for 64 cells only
    B = 16
    forest = omk.Forest.from_soa(soa)
    batch = omk.Batch(forest, B, 4)
    batch.set_roots(np.repeat(roots, B).astype(np.int32))
    with pytest.raises(omk.OmkError):
        batch.leaf_keys(piece, player, np.zeros(B, np.uint64), np.zeros(B, np.int32))   # nothing selected yet
    batch.select(omk.SelectParams(virtual_loss=0))
    _, _, _, actions = batch.read()
    assert actions.max() >= 64
    with pytest.raises(omk.OmkError):
        batch.leaf_keys(piece, player, np.zeros(B, np.uint64), np.zeros(B, np.int32))
