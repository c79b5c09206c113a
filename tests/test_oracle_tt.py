"""The checker's transposition table with the replacement policy against a LITERAL restatement of
PHMapTranspositionTable::store / lookup (reference src/mcts/phmap_transposition_table.cpp:51-117,
createEntry :202-216, Entry::getReplacementScore include/mcts/phmap_transposition_table.h:68-72) over a
Python dict, entry by entry with the same clock (entry i of a call at time t + i).  The two agree
wherever a key occurs once per call or is stored without visits (the reference's two call sites:
the traversal stores unvisited children, the expansion stores distinct leaves); where a call
carries a visited node twice under one key the checker keeps the first, which the test shows too."""
import numpy as np

from oracle import ref_cpu as R


class DictTable:
    """store() and lookup() as written in the reference, the hash map a dict."""

    def __init__(self, threshold=0.1):
        self.e = {}
        self.threshold = np.float32(threshold)

    @staticmethod
    def score(entry, now):
        f = np.float32
        recency = f(1.0) / (f(1.0) + f(np.uint32(now - entry["last_access"])))
        importance = f(entry["visits"]) * (f(1.0) + entry["value"]) * (f(1.0) + f(entry["depth"]))
        return f(recency * importance)

    def store(self, tree, key, node, depth, now):
        n = int(tree.N[node])
        new = dict(node=int(node), depth=int(depth) & 0xFFFF, visits=n,
                   value=np.float32(0.0) if n == 0 else np.float32(tree.W[node]) / np.float32(n), last_access=0)
        old = self.e.get(int(key))
        if old is None:
            self.e[int(key)] = new
            return "new"
        if self.score(new, now) > np.float32(self.score(old, now) * (np.float32(1.0) + self.threshold)):
            self.e[int(key)] = new
            return "replaced"
        return "kept"

    def lookup(self, key, min_depth, now):
        ent = self.e.get(int(key))
        if ent is None or ent["depth"] < min_depth:
            return -1
        ent["last_access"] = int(now)
        return ent["node"]


def tree_with_stats(rng, n):
    N = rng.integers(0, 50, n).astype(np.int32)
    N[rng.random(n) < 0.3] = 0
    W = (rng.uniform(-1, 1, n) * N).astype(np.float32)
    z = np.zeros(n, np.int32)
    return R.RefTree(N=N, W=W, P=np.ones(n, np.float32), VL=z, child_begin=z, child_count=z)


def same_content(tt, table):
    used = tt.slots["key"] != np.uint64(0xFFFFFFFFFFFFFFFF)
    assert int(used.sum()) == len(table.e)
    for s in np.nonzero(used)[0]:
        ent = table.e[int(tt.slots["key"][s])]
        assert (int(tt.slots["node"][s]), int(tt.slots["depth"][s])) == (ent["node"], ent["depth"])
        m = tt.meta[s]
        assert (int(m["visits"]), np.float32(m["value"]), int(m["last_access"])) == (ent["visits"], ent["value"], ent["last_access"])


def test_store_and_lookup_follow_the_literal_restatement():
    rng = np.random.default_rng(1)
    n = 4000
    tree = tree_with_stats(rng, n)
    tt, table = R.RefTT(13), DictTable()
    key_pool = rng.integers(1, 2**63, 1500, dtype=np.uint64)
    replaced = kept = 0
    for call in range(12):
        k = 300
        keys = key_pool[rng.permutation(len(key_pool))[:k]]          # distinct keys within a call
        nodes = rng.integers(0, n, k).astype(np.int32)
        depths = rng.integers(0, 40, k).astype(np.int32)
        t0 = tt.clock
        tt.store(tree, keys, nodes, depths)
        for i in range(k):
            r = table.store(tree, keys[i], nodes[i], depths[i], t0 + i)
            replaced += r == "replaced"
            kept += r == "kept"
        same_content(tt, table)
        # lookups stamp what they find
        probe = np.concatenate([keys[:100], rng.integers(1, 2**63, 50, dtype=np.uint64)])
        for min_depth in (0, 10):
            t0 = tt.clock
            got, hits = tt.lookup(probe, min_depth)
            want = np.array([table.lookup(probe[i], min_depth, t0 + i) for i in range(len(probe))], np.int32)
            assert (got == want).all() and hits == int((want >= 0).sum())
        same_content(tt, table)
        # statistics move between calls, as they do between search steps
        tree.N[rng.integers(0, n, 200)] += 3
    assert replaced > 50 and kept > 50, (replaced, kept)   # both outcomes of the policy were exercised


def test_unvisited_nodes_never_replace_and_first_of_a_call_wins():
    rng = np.random.default_rng(2)
    tree = tree_with_stats(rng, 100)
    tree.N[:10] = 0
    tree.W[:10] = 0.0
    tree.N[10:20] = 7
    tree.W[10:20] = 3.5
    tt, table = R.RefTT(8), DictTable()
    keys = np.arange(1, 6, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15)
    # the traversal's store: nodes without visits, the same key from several traversals in one call
    call_keys = np.concatenate([keys, keys, keys[:2]])
    call_nodes = np.concatenate([np.arange(5), np.arange(5, 10), [3, 4]]).astype(np.int32)
    t0 = tt.clock
    assert tt.store(tree, call_keys, call_nodes, np.full(12, 4, np.int32)) == (5, 0, 7)
    for i in range(12):
        table.store(tree, call_keys[i], call_nodes[i], 4, t0 + i)
    same_content(tt, table)                                   # literal serial order: the same table
    assert (tt.lookup(keys)[0] == np.arange(5)).all()
    # a visited node replaces an unvisited entry (score 0), an unvisited one never replaces anything
    assert tt.store(tree, keys[:2], np.array([12, 2], np.int32), np.array([3, 3], np.int32)) == (0, 1, 0)
    assert tt.lookup(keys[:2])[0].tolist() == [12, 1]
    # a skipped entry (node -1) and a depth beyond 16 bits
    assert tt.store(tree, np.array([77, 78], np.uint64), np.array([-1, 15], np.int32), np.array([1, 65537], np.int32)) == (1, 0, 0)
    assert tt.lookup(np.array([77, 78], np.uint64))[0].tolist() == [-1, 15]
    assert tt.lookup(np.array([78], np.uint64), min_depth=2)[0].tolist() == [-1]      # 65537 was stored as 1
    # where the checker's rule is NOT the literal one: the same key twice in one call, both with visits
    # (the literal order compares the second with the first; the checker drops it)
    assert tt.store(tree, np.array([99, 99], np.uint64), np.array([10, 11], np.int32), np.array([1, 30], np.int32)) == (1, 0, 1)
    assert tt.lookup(np.array([99], np.uint64))[0].tolist() == [10]


def test_traversal_part_reports_transpositions_and_stores_unvisited_children():
    # two paths that reach the same position key by different nodes: 0 -> 1 -> 3 and 0 -> 2 -> 4
    z = np.zeros(5, np.int32)
    tree = R.RefTree(N=np.array([9, 4, 0, 2, 0], np.int32), W=np.zeros(5, np.float32), P=np.ones(5, np.float32), VL=z,
                     child_begin=z, child_count=z)
    paths = np.array([[0, 1, 3], [0, 2, 4], [0, 1, -1]], np.int32)
    plen = np.array([3, 3, 2], np.int32)
    keys = np.array([[11, 50], [12, 50], [11, 0]], np.uint64)       # both second steps stand for position 50
    tt = R.RefTT(6)
    hits, counts = tt.traverse(tree, paths, plen, keys)
    # stored: node 2 (key 12) and node 4 (key 50): the only selected children without visits
    assert counts[:3] == (2, 0, 0)
    assert tt.lookup(np.array([11, 12, 50], np.uint64))[0].tolist() == [-1, 2, 4]
    assert (hits == -1).all() and counts[3] == 0                     # node 4 has no visits: not a transposition
    # after a backup node 4 has visits; the next traversal through node 3 finds it under key 50
    tree.N[4] = 1
    hits, counts = tt.traverse(tree, paths, plen, keys)
    assert hits.tolist() == [[-1, 4], [-1, -1], [-1, -1]] and counts == (0, 0, 0, 1)
