"""Small seeded random trees for parity tests (test-side only)."""
import numpy as np


def star(Np, children, rave=False):
    """Root (id 0) with the given children [N, W, P, VL, raveN, raveW]; returns SoA dict."""
    k = len(children)
    ch = np.asarray(children, dtype=np.float64).reshape(k, -1)
    soa = dict(
        N=np.concatenate([[Np], ch[:, 0]]).astype(np.int32),
        W=np.concatenate([[0.0], ch[:, 1]]).astype(np.float32),
        P=np.concatenate([[0.0], ch[:, 2]]).astype(np.float32),
        VL=np.concatenate([[0], ch[:, 3]]).astype(np.int32),
        child_begin=np.array([1] + [0] * k, dtype=np.int32),
        child_count=np.array([k] + [0] * k, dtype=np.int32),
        action=np.arange(-1, k, dtype=np.int32),
    )
    if rave:
        soa["rN"] = np.concatenate([[0], ch[:, 4]]).astype(np.int32)
        soa["rW"] = np.concatenate([[0.0], ch[:, 5]]).astype(np.float32)
    return soa


def random_tree(seed, n_expand=40, fanout=(1, 12), max_depth=6, n_roots=1, mask_frac=0.0, rave=False,
                zero_frac=0.3, n_max=50, sort_prior=False, vl_frac=0.0, tie_frac=0.0, pad=0):
    """Random CSR forest.  Expansion picks a random unexpanded legal node of depth < max_depth.
    Statistics deliberately include unvisited children, exact ties and pre-existing virtual loss."""
    rng = np.random.default_rng(seed)
    N, W, P, VL, cb, cc, act, depth, legal, rN, rW = ([] for _ in range(11))

    def new_node(d, a, is_legal=True):
        n = 0 if rng.random() < zero_frac else int(rng.integers(1, n_max + 1))
        N.append(n)
        W.append(float(np.float32(rng.uniform(-n, n))) if n else 0.0)
        P.append(0.0)
        VL.append(int(rng.integers(1, 7)) if rng.random() < vl_frac else 0)
        cb.append(0)
        cc.append(0)
        act.append(a)
        depth.append(d)
        legal.append(is_legal)
        r = 0 if rng.random() < zero_frac else int(rng.integers(1, n_max + 1))
        rN.append(r)
        rW.append(float(np.float32(rng.uniform(-r, r))) if r else 0.0)
        return len(N) - 1

    roots = [new_node(0, -1) for _ in range(n_roots)]
    frontier = list(roots)
    for _ in range(n_expand):
        cand = [x for x in frontier if depth[x] < max_depth]
        if not cand:
            break
        node = cand[int(rng.integers(len(cand)))]
        frontier.remove(node)
        f = int(rng.integers(fanout[0], fanout[1] + 1))
        cb[node] = len(N)
        cc[node] = f
        lg = rng.random(f) >= mask_frac
        if not lg.any():
            lg[int(rng.integers(f))] = True
        logits = rng.normal(0, 1.0, f)
        pr = np.where(lg, np.exp(logits), 0.0)
        pr = (pr / pr.sum()).astype(np.float32)
        if sort_prior:
            pr = -np.sort(-pr)
        kids = []
        for i in range(f):
            c = new_node(depth[node] + 1, i, bool(lg[i]))
            P[c] = float(pr[i])
            kids.append(c)
            if lg[i]:
                frontier.append(c)
        if rng.random() < tie_frac and f >= 2:
            # clone the statistics of one child into all its siblings: exact score ties
            s = kids[0]
            for c in kids[1:]:
                N[c], W[c], P[c], VL[c], rN[c], rW[c] = N[s], W[s], P[s], VL[s], rN[s], rW[s]
        N[node] = max(N[node], int(sum(N[c] for c in kids)) + 1)
    for _ in range(pad):
        new_node(0, -1, False)
    n = len(N)
    soa = dict(N=np.array(N, np.int32), W=np.array(W, np.float32), P=np.array(P, np.float32),
               VL=np.array(VL, np.int32), child_begin=np.array(cb, np.int32), child_count=np.array(cc, np.int32),
               action=np.array(act, np.int32))
    if rave:
        soa["rN"] = np.array(rN, np.int32)
        soa["rW"] = np.array(rW, np.float32)
    if mask_frac > 0:
        bits = np.zeros((n + 31) // 32 * 32, dtype=np.uint8)
        bits[:n] = np.array(legal, dtype=np.uint8)
        soa["legal"] = np.packbits(bits.reshape(-1, 32), axis=1, bitorder="little").view("<u4").reshape(-1).copy()
    return soa, np.array(roots, np.int32)


def board_forest(seed, cells=225, root_stones=20, **kw):
    """random_tree whose actions are moves of a stone-placing game on `cells` cells: every root gets a
    random position (root_stones stones, sides alternating, so the side to move follows from the
    parity), and the children of a node play distinct empty cells of the position the node stands
    for.  Returns (soa, roots, root_boards [n_roots, cells] int8 with 0 empty / 1 / 2,
    root_player [n_roots] in {1, 2})."""
    soa, roots = random_tree(seed, **kw)
    rng = np.random.default_rng(seed + 77)
    cb, cc, act = soa["child_begin"], soa["child_count"], soa["action"]
    boards = np.zeros((len(roots), cells), np.int8)
    players = np.zeros(len(roots), np.int32)
    for ri, root in enumerate(roots):
        k = int(rng.integers(0, root_stones + 1))
        for j, c in enumerate(rng.permutation(cells)[:k]):
            boards[ri, c] = 1 + (j & 1)
        players[ri] = 1 + (k & 1)
        stack = [(int(root), set(np.nonzero(boards[ri])[0].tolist()))]
        while stack:
            node, used = stack.pop()
            f = int(cc[node])
            if f == 0:
                continue
            free = np.array(sorted(set(range(cells)) - used))
            picks = rng.permutation(free)[:f]
            assert len(picks) == f
            for i in range(f):
                child = int(cb[node]) + i
                act[child] = int(picks[i])
                stack.append((child, used | {int(picks[i])}))
    return soa, roots, boards, players
