// Batched PUCT selection with virtual loss over the device-resident forest.
//
// What it computes is phase 1 of MCTSEngine::executeBatchedTreeSearch run by ONE thread,
// traversals in index order (reference src/mcts/mcts_engine_batch_tree_simple.cpp:73-185):
// descend while the node is expanded, MCTSNode::selectChild (src/mcts/mcts_node.cpp:90-236),
// addVirtualLoss on the selected child (src/mcts/mcts_node_virtual_loss.cpp:15-20).
//
// How.  During this phase only virtual-loss counters change, and the counter of a child
// matters only to selections made at its parent.  On a tree, the traversals that reach a
// node all come through its parent.  So a work item is (node, the list of traversals that
// reached it, in traversal-index order); ONE 64-lane wavefront owns the item, loads the
// children once (coalesced, one child per lane per round) and plays the visitors in order
// on register-resident statistics: score, DPP arg-max with lowest-index tie-break, bump
// the chosen child's virtual loss, next visitor.  That reproduces the serial order
// exactly.  The visitors are then partitioned by chosen child (stable, so still in
// traversal order) into the work items of the next level's launch; a group that stays
// together (every visitor chose the same child) and a lone visitor are walked on by the
// same wavefront without waiting for that launch.
//
// Playing the visitors of a crowded node one at a time is a chain of dependent wave
// reductions.  The score a child will have after j more visits depends on nothing but j,
// so the lanes evaluate AHEAD: the next E scores of each of the (up to four) children that
// have been winning.  As long as each child's scores do not increase, the serial winner
// sequence is the merge of these descending lists, and every looked-ahead score that
// beats (a) the best score of every other child and (b) the last looked-ahead score of
// each list is certain to be played before anything not evaluated yet.  One round thus
// settles up to 64 visitors with two reductions and a binary-search merge; a round that
// settles nothing falls back to the one-visitor step, so the result never depends on the
// speculation, only the speed does.
#include "omk_internal.h"

namespace omk {

// Register-resident statistics of the children a lane is responsible for: child index
// i = r * 64 + lane for round r.
template <int R, bool RAVE>
struct Kids {
    int n[R];
    float w[R];
    float p[R];
    int vl[R];
    int rn[R];
    float rw[R];
    uint32_t k1[R];
    uint32_t k2[R];
    bool part[R];
};

template <int R, bool RAVE>
__device__ __forceinline__ void load_kids(const ForestDev &f, int cb, int nelig, int lane, Kids<R, RAVE> &k) {
#pragma unroll
    for (int r = 0; r < R; r++) {
        int i = r * kWave + lane;
        bool in = i < nelig;
        int id = cb + i;
        if (in && f.legal) in = (f.legal[(uint32_t)id >> 5] >> ((uint32_t)id & 31u)) & 1u;
        k.part[r] = in;
        k.n[r] = in ? f.N[id] : 0;
        k.w[r] = in ? f.W[id] : 0.0f;
        k.p[r] = in ? f.P[id] : 0.0f;
        k.vl[r] = in ? f.VL[id] : 0;
        if (RAVE) {
            k.rn[r] = in ? f.rN[id] : 0;
            k.rw[r] = in ? f.rW[id] : 0.0f;
        } else {
            k.rn[r] = 0;
            k.rw[r] = 0.0f;
        }
    }
}

template <int R, bool RAVE>
__device__ __forceinline__ void score_round(Kids<R, RAVE> &k, int r, float ep, float rave_k) {
    uint32_t a = 0u, b = 0u;
    if (k.part[r]) child_keys<RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.rn[r], k.rw[r], ep, rave_k, a, b);
    k.k1[r] = a;
    k.k2[r] = b;
}

// Best candidate of this lane in the order (key descending, position ascending); the
// candidates of the second scan sit at positions R*64 + i, after all of the first scan.
// Children whose bit is set in skip are left out.
template <int R, bool RAVE>
__device__ __forceinline__ void lane_best(const Kids<R, RAVE> &k, int lane, uint32_t skip, uint32_t &bk,
                                          uint32_t &bpos) {
    bk = 0u;
    bpos = 0xFFFFFFFFu;
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (k.k1[r] > bk && !((skip >> r) & 1u)) { bk = k.k1[r]; bpos = (uint32_t)(r * kWave + lane); }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (k.k2[r] > bk && !((skip >> r) & 1u)) { bk = k.k2[r]; bpos = (uint32_t)(R * kWave + r * kWave + lane); }
    }
}

// (key, position) of the wave-wide best of per-lane candidates; key 0 = none.
__device__ __forceinline__ void wave_best(uint32_t bk, uint32_t bpos, uint32_t &mk, uint32_t &mpos) {
    mk = wave_max_u32(bk);
    mpos = 0xFFFFFFFFu;
    if (mk != 0u) {
        uint64_t tie = __ballot(bk == mk);
        if (__popcll(tie) == 1) {
            int wl = __builtin_amdgcn_readfirstlane(__ffsll((long long)tie) - 1);
            mpos = (uint32_t)__builtin_amdgcn_readlane((int)bpos, wl);
        } else {
            mpos = wave_min_u32(bk == mk ? bpos : 0xFFFFFFFFu);
        }
    }
}

// Wave-wide winner: child index, or -1 when no child takes part.  When no score beats
// -infinity the reference falls back to the least-visited child, first minimum
// (mcts_node.cpp:173-181).
template <int R, bool RAVE>
__device__ __forceinline__ int wave_pick(const Kids<R, RAVE> &k, int lane, uint32_t bk, uint32_t bpos) {
    uint32_t m, pos;
    wave_best(bk, bpos, m, pos);
    if (m != 0u) return (int)(pos >= (uint32_t)(R * kWave) ? pos - (uint32_t)(R * kWave) : pos);
    uint32_t mn = 0xFFFFFFFFu;  // order-preserving int -> uint
    bool any = false;
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (k.part[r]) {
            any = true;
            mn = umin32(mn, (uint32_t)k.n[r] ^ 0x80000000u);
        }
    }
    if (__ballot(any) == 0ull) return -1;
    uint32_t gm = wave_min_u32(any ? mn : 0xFFFFFFFFu);
    uint32_t idx = 0xFFFFFFFFu;
#pragma unroll
    for (int r = R - 1; r >= 0; r--) {
        if (k.part[r] && ((uint32_t)k.n[r] ^ 0x80000000u) == gm) idx = (uint32_t)(r * kWave + lane);
    }
    return (int)wave_min_u32(idx);
}

struct NodeCtx {
    int cb;
    int cc;
    int nelig;
    float ep;
};

__device__ __forceinline__ NodeCtx node_ctx(const ForestDev &f, const SelectArgs &a, int node, int np) {
    NodeCtx c;
    int2 sp = f.span[node];
    c.cb = sp.x;
    c.cc = sp.y;
    c.nelig = c.cc;
    if (a.pw) {
        int kk = ceil_sqrt_i32(np);
        c.nelig = kk < c.cc ? kk : c.cc;
    }
    c.ep = a.c_puct * sqrtf((float)np);
    return c;
}

// One selection for a single visitor.  Returns the child index or -1; np_child receives
// the visit count of the chosen child (the next node's N_parent).
template <int R, bool RAVE>
__device__ __forceinline__ int select_single(const ForestDev &f, const SelectArgs &a, const NodeCtx &c, int lane,
                                             int &np_child) {
    Kids<R, RAVE> k;
    load_kids<R, RAVE>(f, c.cb, c.nelig, lane, k);
#pragma unroll
    for (int r = 0; r < R; r++) score_round<R, RAVE>(k, r, c.ep, a.rave_k);
    uint32_t bk, bpos;
    lane_best<R, RAVE>(k, lane, 0u, bk, bpos);
    int i = wave_pick<R, RAVE>(k, lane, bk, bpos);
    if (i < 0) return -1;
    int nsel = 0;
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (r == (i >> 6)) nsel = k.n[r];
    }
    np_child = __builtin_amdgcn_readlane(nsel, i & 63);
    return i;
}

// The children that have been winning lately, with a wave-uniform copy of their current
// statistics so that any lane can evaluate their future scores.
struct Dominant {
    int child[4];
    int n[4];
    float w[4];
    float p[4];
    int vl[4];  // current counter, picks of this item included
    int rn[4];
    float rw[4];
    int cnt[4];  // picks of this item so far
    int stale[4];
    int K;
};

// Where the walk goes on after a multi-visitor node whose visitors all chose one child.
struct Continuation {
    int node;
    int off;
    int m;
    int np;
};

// All visitors of a multi-visitor item, in order.  Records the chosen child of every
// visitor, bumps virtual loss, partitions the visitors by child into seg_out, writes the
// next path entry, appends one item per visited child to the next level's queue (none when
// all visitors chose the same child: then the caller walks on with them).  Returns false when no child takes part in the selection.
template <int R, bool RAVE>
__device__ __forceinline__ bool select_group(const ForestDev &f, const SelectArgs &a, const NodeCtx &c, int lane,
                                             const int32_t *seg_in, int32_t *seg_out, int off, int m, int depth,
                                             int *s_offs, Continuation &next) {
    Kids<R, RAVE> k;
    int cnt[R];
    load_kids<R, RAVE>(f, c.cb, c.nelig, lane, k);
#pragma unroll
    for (int r = 0; r < R; r++) {
        score_round<R, RAVE>(k, r, c.ep, a.rave_k);
        cnt[r] = 0;
    }
    uint32_t bk, bpos;
    lane_best<R, RAVE>(k, lane, 0u, bk, bpos);

    Dominant dom;
    dom.K = 0;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        dom.child[g] = -1;
        dom.n[g] = 0;
        dom.w[g] = 0.0f;
        dom.p[g] = 0.0f;
        dom.vl[g] = 0;
        dom.rn[g] = 0;
        dom.rw[g] = 0.0f;
        dom.cnt[g] = 0;
        dom.stale[g] = 0;
    }
    uint32_t dmask = 0u;  // bit r: child r*64+lane is in the dominant set
    int done = 0;
    int backoff = 0;
    int fails = 0;
    int recent0 = -1, recent1 = -1;  // the last two children settled one at a time
    int st_rounds = 0, st_settled = 0, st_single = 0, st_viol = 0, st_none = 0;
    const uint32_t uvl = a.vl > 0 ? (uint32_t)a.vl : 0u;

    while (done < m) {
        if (dom.K > 0 && backoff == 0 && m - done >= 4) {
            // ---- look-ahead round ----
            const int K = dom.K;
            st_rounds++;
            const int logE = K <= 1 ? 6 : (K == 2 ? 5 : 4);
            const int E = 1 << logE;
            const int g = lane >> logE;
            const int o = lane & (E - 1);
            const bool slot = g < K;
            int sc = -1, sn = 0, svl = 0, srn = 0, scnt = 0;
            float sw = 0.0f, sp = 0.0f, srw = 0.0f;
#pragma unroll
            for (int gg = 0; gg < 4; gg++) {
                if (g == gg) {
                    sc = dom.child[gg];
                    sn = dom.n[gg];
                    sw = dom.w[gg];
                    sp = dom.p[gg];
                    svl = dom.vl[gg];
                    srn = dom.rn[gg];
                    srw = dom.rw[gg];
                    scnt = dom.cnt[gg];
                }
            }
            uint32_t ek = 0u, epos = 0xFFFFFFFFu, ek1 = 0u, ek2 = 0u;
            if (slot) {
                int vlj = (int)((uint32_t)svl + (uint32_t)o * uvl);
                child_keys<RAVE>(sn, sw, sp, vlj, srn, srw, c.ep, a.rave_k, ek1, ek2);
                if (ek2 > ek1) {
                    ek = ek2;
                    epos = (uint32_t)(R * kWave + sc);
                } else {
                    ek = ek1;
                    epos = (uint32_t)sc;
                }
            }
            // each list must not increase in the order (key descending, position ascending)
            uint32_t pk = (uint32_t)__shfl_up((int)ek, 1, kWave);
            uint32_t ppos = (uint32_t)__shfl_up((int)epos, 1, kWave);
            bool viol = slot && o > 0 && ek != 0u && (pk == 0u || ek > pk || (ek == pk && epos < ppos));
            bool ok = __ballot(viol) == 0ull;
            if (!ok) st_viol++;
            int settled = 0;
            if (ok) {
                // bound: best head of every other child, and the last evaluated entry of each list
                uint32_t ck, cpos;
                lane_best<R, RAVE>(k, lane, dmask, ck, cpos);
                if (slot && o == E - 1 && ek != 0u && (ek > ck || (ek == ck && epos < cpos))) {
                    ck = ek;
                    cpos = epos;
                }
                uint32_t tk, tpos;
                wave_best(ck, cpos, tk, tpos);
                bool acc = slot && ek != 0u && (ek > tk || (ek == tk && epos < tpos));
                uint64_t accm = __ballot(acc);
                if (accm != 0ull) {
                    // rank in the merged order: own offset + entries of the other lists that come first
                    int rank = o;
                    if (K > 1) {
                        // binary searches in the other lists, advanced together so that their
                        // cross-lane reads overlap
                        int lo[4], hi[4];
#pragma unroll
                        for (int gg = 0; gg < 4; gg++) {
                            lo[gg] = 0;
                            hi[gg] = E;
                        }
                        for (int s = 0; s <= logE; s++) {
                            uint32_t mk[4], mpos[4];
#pragma unroll
                            for (int gg = 0; gg < 4; gg++) {
                                if (gg < K) {
                                    int mid = (lo[gg] + hi[gg]) >> 1;
                                    int src = (gg << logE) + (mid < E ? mid : E - 1);
                                    mk[gg] = (uint32_t)__shfl((int)ek, src, kWave);
                                    mpos[gg] = (uint32_t)__shfl((int)epos, src, kWave);
                                }
                            }
#pragma unroll
                            for (int gg = 0; gg < 4; gg++) {
                                if (gg < K && lo[gg] < hi[gg]) {
                                    int mid = (lo[gg] + hi[gg]) >> 1;
                                    bool before = mk[gg] != 0u && (mk[gg] > ek || (mk[gg] == ek && mpos[gg] < epos));
                                    if (before) lo[gg] = mid + 1;
                                    else hi[gg] = mid;
                                }
                            }
                        }
#pragma unroll
                        for (int gg = 0; gg < 4; gg++)
                            if (gg < K && gg != g) rank += lo[gg];
                    }
                    const int remaining = m - done;
                    const bool valid = acc && rank < remaining;
                    if (valid) {
                        a.sc_child[off + done + rank] = sc;
                        a.sc_occ[off + done + rank] = scnt + o;
                    }
#pragma unroll
                    for (int gg = 0; gg < 4; gg++) {
                        if (gg < K) {
                            int ag = __popcll(__ballot(valid && g == gg));
                            if (ag > 0) {
                                dom.stale[gg] = 0;
                                dom.vl[gg] = (int)((uint32_t)dom.vl[gg] + (uint32_t)ag * uvl);
                                dom.cnt[gg] += ag;
                                int ch = dom.child[gg];
                                // the new head of this child was looked ahead at offset ag
                                // (the last entry of a list is never settled, so ag < E)
                                const int hl = (gg << logE) + ag;
                                uint32_t nk1 = (uint32_t)__builtin_amdgcn_readlane((int)ek1, hl);
                                uint32_t nk2 = (uint32_t)__builtin_amdgcn_readlane((int)ek2, hl);
                                if (lane == (ch & 63)) {
#pragma unroll
                                    for (int r = 0; r < R; r++) {
                                        if (r == (ch >> 6)) {
                                            cnt[r] += ag;
                                            k.vl[r] = (int)((uint32_t)k.vl[r] + (uint32_t)ag * uvl);
                                            k.k1[r] = nk1;
                                            k.k2[r] = nk2;
                                        }
                                    }
                                }
                            } else {
                                dom.stale[gg]++;
                            }
                        }
                    }
                    lane_best<R, RAVE>(k, lane, 0u, bk, bpos);
                    int A = __popcll(accm);
                    settled = A < remaining ? A : remaining;
                    // lists that stopped winning leave the set (more look-ahead for the others):
                    // the last list moves into the freed place
#pragma unroll
                    for (int gg = 3; gg >= 0; gg--) {
                        if (gg < dom.K && dom.stale[gg] >= 2) {
                            int ch = dom.child[gg];
                            if (lane == (ch & 63)) dmask &= ~(1u << (ch >> 6));
                            const int last = dom.K - 1;
                            int mc = -1, mn = 0, mvl = 0, mrn = 0, mcnt = 0, mst = 0;
                            float mw = 0.0f, mp = 0.0f, mrw = 0.0f;
#pragma unroll
                            for (int q = 0; q < 4; q++) {
                                if (q == last) {
                                    mc = dom.child[q];
                                    mn = dom.n[q];
                                    mw = dom.w[q];
                                    mp = dom.p[q];
                                    mvl = dom.vl[q];
                                    mrn = dom.rn[q];
                                    mrw = dom.rw[q];
                                    mcnt = dom.cnt[q];
                                    mst = dom.stale[q];
                                }
                            }
                            dom.child[gg] = mc;
                            dom.n[gg] = mn;
                            dom.w[gg] = mw;
                            dom.p[gg] = mp;
                            dom.vl[gg] = mvl;
                            dom.rn[gg] = mrn;
                            dom.rw[gg] = mrw;
                            dom.cnt[gg] = mcnt;
                            dom.stale[gg] = mst;
                            dom.K = last;
                        }
                    }
                }
            }
            if (settled > 0) {
                done += settled;
                st_settled += settled;
                fails = 0;
                continue;
            }
            if (ok) st_none++;
            fails = fails < 5 ? fails + 1 : 5;
            backoff = 1 << fails;
        }

        // ---- one visitor ----
        int i = wave_pick<R, RAVE>(k, lane, bk, bpos);
        if (i < 0) return false;  // no child takes part: uniform, and then for every visitor
        st_single++;
        int tn = 0, tvl = 0, trn = 0, tcnt = 0;
        float tw = 0.0f, tp = 0.0f, trw = 0.0f;
        if (lane == (i & 63)) {
            int occ = 0;
#pragma unroll
            for (int r = 0; r < R; r++) {
                if (r == (i >> 6)) {
                    occ = cnt[r];
                    cnt[r] = occ + 1;
                    k.vl[r] = (int)((uint32_t)k.vl[r] + uvl);
                    score_round<R, RAVE>(k, r, c.ep, a.rave_k);
                    tn = k.n[r];
                    tw = k.w[r];
                    tp = k.p[r];
                    tvl = k.vl[r];
                    trn = k.rn[r];
                    trw = k.rw[r];
                    tcnt = cnt[r];
                }
            }
            lane_best<R, RAVE>(k, lane, 0u, bk, bpos);
            a.sc_child[off + done] = i;
            a.sc_occ[off + done] = occ;
        }
        done++;
        if (a.vl <= 0) {
            // no virtual loss: nothing changes between visitors, they all follow the first
            for (int j = done + lane; j < m; j += kWave) {
                a.sc_child[off + j] = i;
                a.sc_occ[off + j] = j;
            }
            if (lane == (i & 63)) {
#pragma unroll
                for (int r = 0; r < R; r++)
                    if (r == (i >> 6)) cnt[r] = m;
            }
            done = m;
            break;
        }
        if (backoff > 0) backoff--;
        // keep the dominant set current
        int found = -1;
#pragma unroll
        for (int gg = 0; gg < 4; gg++)
            if (gg < dom.K && dom.child[gg] == i) found = gg;
        if (found >= 0) {
#pragma unroll
            for (int gg = 0; gg < 4; gg++) {
                if (gg == found) {
                    dom.vl[gg] = (int)((uint32_t)dom.vl[gg] + uvl);
                    dom.cnt[gg] += 1;
                    dom.stale[gg] = 0;
                }
            }
        } else if (i == recent0 || i == recent1) {
            int slot_g = dom.K;
            if (dom.K >= 4) {
                slot_g = 0;
                int worst = dom.stale[0];
#pragma unroll
                for (int gg = 1; gg < 4; gg++) {
                    if (dom.stale[gg] >= worst) {
                        worst = dom.stale[gg];
                        slot_g = gg;
                    }
                }
                int ev = -1;
#pragma unroll
                for (int gg = 0; gg < 4; gg++)
                    if (gg == slot_g) ev = dom.child[gg];
                if (lane == (ev & 63)) dmask &= ~(1u << (ev >> 6));
            } else {
                dom.K++;
            }
            const int ol = i & 63;
            int xn = __builtin_amdgcn_readlane(tn, ol);
            float xw = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tw), ol));
            float xp = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tp), ol));
            int xvl = __builtin_amdgcn_readlane(tvl, ol);
            int xrn = __builtin_amdgcn_readlane(trn, ol);
            float xrw = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(trw), ol));
            int xcnt = __builtin_amdgcn_readlane(tcnt, ol);
#pragma unroll
            for (int gg = 0; gg < 4; gg++) {
                if (gg == slot_g) {
                    dom.child[gg] = i;
                    dom.n[gg] = xn;
                    dom.w[gg] = xw;
                    dom.p[gg] = xp;
                    dom.vl[gg] = xvl;
                    dom.rn[gg] = xrn;
                    dom.rw[gg] = xrw;
                    dom.cnt[gg] = xcnt;
                    dom.stale[gg] = 0;
                }
            }
            if (lane == ol) dmask |= 1u << (i >> 6);
        }
        recent1 = recent0;
        recent0 = i;
    }

    if (a.stats && lane == 0) {
        atomicAdd(a.stats + 0, 1);
        atomicAdd(a.stats + 1, st_rounds);
        atomicAdd(a.stats + 2, st_settled);
        atomicAdd(a.stats + 3, st_single);
        atomicAdd(a.stats + 4, st_viol);
        atomicAdd(a.stats + 5, st_none);
    }
    // the child with most visitors (lowest index on ties) is where this wavefront walks on
    uint32_t lmax = 0u;
#pragma unroll
    for (int r = 0; r < R; r++) lmax = umax32(lmax, (uint32_t)cnt[r]);
    const uint32_t gmax = wave_max_u32(lmax);
    uint32_t lidx = 0xFFFFFFFFu;
#pragma unroll
    for (int r = R - 1; r >= 0; r--)
        if ((uint32_t)cnt[r] == gmax) lidx = (uint32_t)(r * kWave + lane);
    // walking on is only worth it when the group stays together: a split group is handed to
    // the next level's launch whole, so that its parts are played side by side
    const int keep = gmax == (uint32_t)m ? (int)wave_min_u32(lidx) : -1;

    // exclusive prefix of the visit counts in child order -> segment of every child
    int carry = 0;
    int keep_np = 0;
#pragma unroll
    for (int r = 0; r < R; r++) {
        int inc = wave_inclusive_sum(cnt[r], lane);
        int excl = carry + inc - cnt[r];
        int i = r * kWave + lane;
        s_offs[i] = excl;
        if (i == keep) keep_np = k.n[r];
        uint64_t has = __ballot(cnt[r] > 0 && i != keep);
        int nnew = __popcll(has);
        if (nnew > 0) {
            int slot0 = 0;
            if (lane == 0) slot0 = atomicAdd(a.counters + depth + 1, nnew);
            slot0 = __builtin_amdgcn_readfirstlane(slot0);
            if (cnt[r] > 0 && i != keep) {
                int slot = slot0 + __popcll(has & ((1ull << lane) - 1ull));
                Item it;
                it.node = c.cb + i;
                it.off = off + excl;
                it.m = cnt[r];
                it.np = k.n[r];
                a.items_q[(size_t)depth * a.stride + slot] = it;
            }
        }
        if (cnt[r] > 0 && a.vl > 0) atomicAdd(f.VL + c.cb + i, (int)((uint32_t)a.vl * (uint32_t)cnt[r]));
        carry += __builtin_amdgcn_readlane(inc, 63);
    }
    // make this wave's LDS and scratch writes visible to its own other lanes
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    int *path_next = a.paths + (size_t)(depth + 1) * a.stride;
    for (int j = lane; j < m; j += kWave) {
        int t = seg_in[off + j];
        int i = a.sc_child[off + j];
        path_next[t] = c.cb + i;
        seg_out[off + s_offs[i] + a.sc_occ[off + j]] = t;
    }
    next.node = -1;
    if (keep >= 0) {
        next.node = c.cb + keep;
        next.off = off + s_offs[keep];
        next.m = (int)gmax;
        next.np = __builtin_amdgcn_readlane(keep_np, keep & 63);
    }
    // the next step of the walk reads seg_out and reuses s_offs
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    return true;
}

template <int RMAX, bool RAVE>
__global__ __launch_bounds__(256) void k_select_level(ForestDev f, SelectArgs a, int level) {
    __shared__ int s_offs_all[4][RMAX * kWave];
    const int lane = threadIdx.x & 63;
    const int wib = threadIdx.x >> 6;
    const int wave = blockIdx.x * 4 + wib;
    if (wave >= a.counters[level]) return;
    const Item it = level == 0 ? a.items0[wave] : a.items_q[(size_t)(level - 1) * a.stride + wave];
    int node = it.node;
    int np = level == 0 ? f.N[node] : it.np;
    int off = it.off;
    int m = it.m;
    int depth = level;
    if (level == 0) {
        for (int j = lane; j < m; j += kWave) a.paths[a.seg0[off + j]] = node;
    }

    // walk with a group of visitors while there is more than one
    while (m > 1) {
        const int32_t *seg_in = depth == 0 ? a.seg0 : a.seg[(depth - 1) & 1];
        int32_t *seg_out = a.seg[depth & 1];
        NodeCtx c = node_ctx(f, a, node, np);
        bool descended = false;
        Continuation next;
        if (c.cc > 0 && depth < a.max_depth) {
            int *s_offs = s_offs_all[wib];
            if (c.cc <= kWave)
                descended = select_group<1, RAVE>(f, a, c, lane, seg_in, seg_out, off, m, depth, s_offs, next);
            else
                descended = select_group<RMAX, RAVE>(f, a, c, lane, seg_in, seg_out, off, m, depth, s_offs, next);
        }
        if (!descended) {
            for (int j = lane; j < m; j += kWave) {
                int t = seg_in[off + j];
                a.leaf[t] = node;
                a.path_len[t] = depth + 1;
            }
            if (c.cc > 0 && depth >= a.max_depth && lane == 0) atomicAdd(a.truncated, m);
            return;
        }
        if (next.node < 0) return;
        node = next.node;
        off = next.off;
        m = next.m;
        np = next.np;
        depth++;
    }

    // single visitor: the rest of the path is private to it
    const int32_t *seg_in = depth == 0 ? a.seg0 : a.seg[(depth - 1) & 1];
    const int t = seg_in[off];
    int d = depth;
    for (;;) {
        NodeCtx c = node_ctx(f, a, node, np);
        int i = -1;
        int np_child = 0;
        if (c.cc > 0 && d < a.max_depth) {
            if (c.cc <= kWave) i = select_single<1, RAVE>(f, a, c, lane, np_child);
            else i = select_single<RMAX, RAVE>(f, a, c, lane, np_child);
        }
        if (i < 0) {
            if (lane == 0) {
                a.leaf[t] = node;
                a.path_len[t] = d + 1;
                if (c.cc > 0 && d >= a.max_depth) atomicAdd(a.truncated, 1);
            }
            return;
        }
        int child = c.cb + i;
        if (lane == 0) {
            if (a.stats) atomicAdd(a.stats + 6, 1);
            if (a.vl > 0) atomicAdd(f.VL + child, a.vl);
            a.paths[(size_t)(d + 1) * a.stride + t] = child;
        }
        node = child;
        np = np_child;
        d++;
    }
}

__global__ void k_select_reset(int *counters, int n_counters, int n_items0, int *truncated, int *stats) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_counters) counters[i] = (i == 0) ? n_items0 : 0;
    if (i == 0) *truncated = 0;
    if (stats && i < 8) stats[i] = 0;
}

template <int RMAX, bool RAVE>
static hipError_t launch_levels(const ForestDev &f, const SelectArgs &a, int n_traversals, hipStream_t s) {
    const int grid = (n_traversals + 3) / 4;
    for (int level = 0; level <= a.max_depth; level++)
        hipLaunchKernelGGL((k_select_level<RMAX, RAVE>), dim3(grid), dim3(256), 0, s, f, a, level);
    return hipGetLastError();
}

hipError_t launch_select(const ForestDev &f, const SelectArgs &a, int n_items0, int n_traversals, int max_fanout,
                         bool rave, hipStream_t s) {
    hipLaunchKernelGGL(k_select_reset, dim3((a.max_depth + 2 + 63) / 64), dim3(64), 0, s, a.counters,
                       a.max_depth + 2, n_items0, a.truncated, a.stats);
#define OMK_DISPATCH(RM) \
    return rave ? launch_levels<RM, true>(f, a, n_traversals, s) : launch_levels<RM, false>(f, a, n_traversals, s)
    if (max_fanout <= 64) { OMK_DISPATCH(1); }
    if (max_fanout <= 256) { OMK_DISPATCH(4); }
    if (max_fanout <= 384) { OMK_DISPATCH(6); }
    OMK_DISPATCH(16);
#undef OMK_DISPATCH
}

}  // namespace omk
