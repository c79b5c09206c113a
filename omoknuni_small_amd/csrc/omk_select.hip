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
// reached it, in traversal-index order); ONE 64-lane wavefront owns the item and loads the
// children once (coalesced, one child per lane per round).  The visitors are then
// partitioned by chosen child (stable, so still in traversal order) into the work items
// of the next level's launch; a group that stays together (every visitor chose the same
// child) and a lone visitor are walked on by the same wavefront.
//
// Which child each visitor chooses:
//  * few visitors: they are played one after another on register-resident statistics --
//    score, DPP arg-max with lowest-index tie-break, bump the chosen child's virtual loss,
//    next visitor.  That is the serial order itself.
//  * many visitors ("water level"): the score child i shows to its j-th visitor of this
//    batch depends on nothing but j.  If every child's scores do not increase with j, the
//    serial winner sequence is the merge of these descending lists, i.e. the m best
//    entries (i, j) in the order (score descending, candidate position ascending, j
//    ascending).  A bisection on the score threshold finds how many entries each child
//    contributes, all m entries are evaluated in parallel, a stable radix sort puts them
//    in winner order.  Nothing is assumed: afterwards the wavefront checks, on the exact
//    binary32 values, (i) that every child's taken entries and its first untaken entry do
//    not increase and (ii) that the last taken entry still comes before every child's
//    first untaken one.  Under (i) and (ii) the serial loop provably produces exactly
//    this sequence; if either fails the node is replayed one visitor at a time.
#include "omk_internal.h"

namespace omk {

constexpr int kRunMin = 4;                // visitors from which the one-winner check is tried
constexpr int kWaterLevelMin = 32;        // visitors from which the parallel path is tried
constexpr int kWaterLevelMaxJ = 1 << 21;  // entries per child representable in the sort payload

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

// Per-wavefront scratch in LDS.
template <int R>
struct WaveLds {
    int offs[R * kWave];  // exclusive prefix of the visit counts in child order
    int st_n[R * kWave];
    float st_w[R * kWave];
    float st_p[R * kWave];
    int st_vl[R * kWave];
    int st_rn[R * kWave];
    float st_rw[R * kWave];
    int hist[256];
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
template <int R, bool RAVE>
__device__ __forceinline__ void lane_best(const Kids<R, RAVE> &k, int lane, uint32_t &bk, uint32_t &bpos) {
    bk = 0u;
    bpos = 0xFFFFFFFFu;
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (k.k1[r] > bk) { bk = k.k1[r]; bpos = (uint32_t)(r * kWave + lane); }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (k.k2[r] > bk) { bk = k.k2[r]; bpos = (uint32_t)(R * kWave + r * kWave + lane); }
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
    lane_best<R, RAVE>(k, lane, bk, bpos);
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

// Key and candidate position child `child` shows to its j-th visitor of this batch.
template <int R, bool RAVE>
__device__ __forceinline__ void entry_key(int n, float w, float p, int vl0, int rn, float rw, float ep,
                                          float rave_k, uint32_t uvl, int j, int child, uint32_t &key,
                                          uint32_t &pos) {
    int vlj = (int)((uint32_t)vl0 + (uint32_t)j * uvl);
    uint32_t k1, k2;
    child_keys<RAVE>(n, w, p, vlj, rn, rw, ep, rave_k, k1, k2);
    if (k2 > k1) {
        key = k2;
        pos = (uint32_t)(R * kWave + child);
    } else {
        key = k1;
        pos = (uint32_t)child;
    }
}

// true when candidate (ka, pa) is played strictly before candidate (kb, pb)
__device__ __forceinline__ bool comes_before(uint32_t ka, uint32_t pa, uint32_t kb, uint32_t pb) {
    return ka > kb || (ka == kb && pa < pb);
}

__device__ __forceinline__ void wave_sync_memory() {
    // Orders this wavefront's LDS / global writes before its own later reads from other
    // lanes.  One wavefront's memory operations reach the cache in program order, so this
    // only has to stop the compiler from moving them across.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The visitors of a crowded node, all at once (see the file header).  On success cnt[r]
// holds the visitors of every child and sc_child / sc_occ hold (child, visit number) of
// every visitor; returns false, having changed nothing that matters, when the node has to
// be replayed one visitor at a time.
template <int R, bool RAVE>
__device__ __forceinline__ bool water_level(const SelectArgs &a, const NodeCtx &c, int lane, const Kids<R, RAVE> &k,
                                            uint32_t bk, uint32_t bpos, int off, int m, WaveLds<R> &lds,
                                            int (&cnt)[R]) {
    constexpr int F = R * kWave;
    const uint32_t uvl = (uint32_t)a.vl;
    if (m > kWaterLevelMaxJ) return false;

    // ---- 1. threshold T* = largest key with at least m entries at or above it ----
    uint32_t hi_key, hi_pos;
    wave_best(bk, bpos, hi_key, hi_pos);
    if (hi_key == 0u) return false;
    const int best = (int)(hi_pos >= (uint32_t)F ? hi_pos - (uint32_t)F : hi_pos);
    // the best child alone has m entries at or above the key of its m-th visit
    uint32_t lo_key = 0u;
    {
        uint32_t kk = 0u, pp = 0u;
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (r == (best >> 6))
                entry_key<R, RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.rn[r], k.rw[r], c.ep, a.rave_k, uvl, m - 1,
                                   best, kk, pp);
        }
        lo_key = (uint32_t)__builtin_amdgcn_readlane((int)kk, best & 63);
    }
    if (lo_key == 0u) lo_key = 1u;
    if (lo_key > hi_key) return false;  // scores rose along the best child's list

    int cl[R], ch[R];
    uint32_t head[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        head[r] = umax32(k.k1[r], k.k2[r]);
        cl[r] = 0;
        ch[r] = head[r] != 0u ? m : 0;
    }
    // Invariant: count(lo) >= m > count(hi), cl = per-child counts at hi, ch = at lo.  After
    // every probe the bracket end that moved is snapped to the nearest key that actually
    // occurs, so the search ends after about log2(distinct keys in the bracket) probes.
    uint32_t lo = lo_key, hi = hi_key + 1u;
    bool first = true;
    int probes = 0;
    while (first || hi - lo > 1u) {
        if (++probes > 80) return false;
        const uint32_t T = first ? lo : lo + ((hi - lo) >> 1);
        int ct[R];
        int sum = 0;
        uint32_t below = 0u;             // largest key below T among the first entries below T
        uint32_t above = 0xFFFFFFFFu;    // smallest key at or above T among the last entries at or above T
#pragma unroll
        for (int r = 0; r < R; r++) {
            int lo_c = cl[r], hi_c = ch[r];
            if (head[r] < T) hi_c = 0;  // a list that starts below T has nothing above it
            if (lo_c > hi_c) lo_c = hi_c;
            uint32_t k_in = 0xFFFFFFFFu, k_out = 0u;  // keys seen at the boundary while searching
            int j_in = -1, j_out = -1;
            while (lo_c < hi_c) {
                int t = (lo_c + hi_c + 1) >> 1;
                uint32_t kk, pp;
                entry_key<R, RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.rn[r], k.rw[r], c.ep, a.rave_k, uvl, t - 1,
                                   r * kWave + lane, kk, pp);
                if (kk >= T) {
                    lo_c = t;
                    k_in = kk;
                    j_in = t - 1;
                } else {
                    hi_c = t - 1;
                    k_out = kk;
                    j_out = t - 1;
                }
            }
            ct[r] = lo_c;
            sum = sum + lo_c > m ? m : sum + lo_c;
            if (head[r] != 0u) {
                // last entry at or above T and first entry below T of this child
                if (lo_c > 0) {
                    if (j_in != lo_c - 1) {
                        if (lo_c == 1) {
                            k_in = head[r];
                        } else {
                            uint32_t pp;
                            entry_key<R, RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.rn[r], k.rw[r], c.ep, a.rave_k, uvl,
                                               lo_c - 1, r * kWave + lane, k_in, pp);
                        }
                    }
                    above = umin32(above, k_in);
                }
                if (lo_c < m) {
                    if (j_out != lo_c) {
                        if (lo_c == 0) {
                            k_out = head[r];
                        } else {
                            uint32_t pp;
                            entry_key<R, RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.rn[r], k.rw[r], c.ep, a.rave_k, uvl,
                                               lo_c, r * kWave + lane, k_out, pp);
                        }
                    }
                    if (k_out < T) below = umax32(below, k_out);
                }
            }
        }
        const int total = wave_sum_i32(sum);  // at most 64 * m
        if (first) {
            if (total < m) return false;
            first = false;
        }
        if (total >= m) {
            uint32_t snap = wave_min_u32(above);
            lo = (snap != 0xFFFFFFFFu && snap >= T && snap < hi) ? snap : T;
#pragma unroll
            for (int r = 0; r < R; r++) ch[r] = ct[r];
        } else {
            uint32_t snap = wave_max_u32(below);
            hi = (snap + 1u > lo && snap < T) ? snap + 1u : T;
#pragma unroll
            for (int r = 0; r < R; r++) cl[r] = ct[r];
        }
    }
    // now cl = entries above T*, ch = entries at or above T*

    // ---- 2. entries at exactly T* are handed out in child order until m is reached ----
    int above = 0;
#pragma unroll
    for (int r = 0; r < R; r++) above = above + cl[r] > m ? m : above + cl[r];
    int rem = m - wave_sum_i32(above);
    if (rem < 0) return false;
    int cv[R];
    int carry = 0;
#pragma unroll
    for (int r = 0; r < R; r++) {
        int e = ch[r] - cl[r];
        if (e < 0) e = 0;
        if (e > rem) e = rem;
        int inc = wave_inclusive_sum(e, lane);
        long long excl = (long long)carry + inc - e;
        long long left = (long long)rem - excl;
        int take = left <= 0 ? 0 : (left < e ? (int)left : e);
        cv[r] = cl[r] + take;
        int tot = __builtin_amdgcn_readlane(inc, 63);
        carry = carry + tot > m ? m : carry + tot;
    }
    int csum = 0;
#pragma unroll
    for (int r = 0; r < R; r++) csum = csum + cv[r] > m + 1 ? m + 1 : csum + cv[r];
    if (wave_sum_i32(csum) != m) return false;

    // ---- 3. evaluate the m entries, in (child, visit) order; first untaken entries ----
    carry = 0;
    uint32_t uk[R], upos[R];  // first untaken entry of every child of this lane
    bool bad = false;
#pragma unroll
    for (int r = 0; r < R; r++) {
        int inc = wave_inclusive_sum(cv[r], lane);
        int i = r * kWave + lane;
        lds.offs[i] = carry + inc - cv[r];
        lds.st_n[i] = k.n[r];
        lds.st_w[i] = k.w[r];
        lds.st_p[i] = k.p[r];
        lds.st_vl[i] = k.vl[r];
        if (RAVE) {
            lds.st_rn[i] = k.rn[r];
            lds.st_rw[i] = k.rw[r];
        }
        carry += __builtin_amdgcn_readlane(inc, 63);
        uk[r] = 0u;
        upos[r] = 0xFFFFFFFFu;
        if (k.part[r]) {
            uint32_t kk, pp;
            entry_key<R, RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.rn[r], k.rw[r], c.ep, a.rave_k, uvl, cv[r], i, kk,
                               pp);
            uk[r] = kk;
            upos[r] = pp;
            if (cv[r] > 0) {
                // the last taken entry of the child must not come after its first untaken one
                uint32_t lk, lp;
                entry_key<R, RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.rn[r], k.rw[r], c.ep, a.rave_k, uvl,
                                   cv[r] - 1, i, lk, lp);
                if (lk == 0u || comes_before(kk, pp, lk, lp)) bad = true;
            }
        }
    }
    wave_sync_memory();

    uint32_t *keyA = (uint32_t *)a.sort_key[0] + off, *keyB = (uint32_t *)a.sort_key[1] + off;
    uint32_t *payA = (uint32_t *)a.sort_pay[0] + off, *payB = (uint32_t *)a.sort_pay[1] + off;
    uint32_t kmin = 0xFFFFFFFFu, kmax = 0u;
    uint32_t prev_key63 = 0u, prev_pos63 = 0u;
    int prev_child63 = -1;
    for (int base = 0; base < m; base += kWave) {
        const int q = base + lane;
        const bool in = q < m;
        int child = -1;
        uint32_t kk = 0u, pp = 0u;
        if (in) {
            // last child whose segment starts at or before q
            int lo_i = 0, hi_i = F;
            while (hi_i - lo_i > 1) {
                int mid = (lo_i + hi_i) >> 1;
                if (lds.offs[mid] <= q) lo_i = mid;
                else hi_i = mid;
            }
            child = lo_i;
            const int j = q - lds.offs[child];
            entry_key<R, RAVE>(lds.st_n[child], lds.st_w[child], lds.st_p[child], lds.st_vl[child],
                               RAVE ? lds.st_rn[child] : 0, RAVE ? lds.st_rw[child] : 0.0f, c.ep, a.rave_k, uvl, j,
                               child, kk, pp);
            keyA[q] = ~kk;
            payA[q] = (pp >= (uint32_t)F ? 0x80000000u : 0u) | ((uint32_t)child << 21) | (uint32_t)j;
            kmin = umin32(kmin, ~kk);
            kmax = umax32(kmax, ~kk);
            if (kk == 0u) bad = true;
        }
        // within a child the entries must not increase
        uint32_t pk = (uint32_t)__shfl_up((int)kk, 1, kWave);
        uint32_t ppos = (uint32_t)__shfl_up((int)pp, 1, kWave);
        int pchild = __shfl_up(child, 1, kWave);
        if (lane == 0) {
            pk = prev_key63;
            ppos = prev_pos63;
            pchild = prev_child63;
        }
        if (in && pchild == child && comes_before(kk, pp, pk, ppos)) bad = true;
        prev_key63 = (uint32_t)__builtin_amdgcn_readlane((int)kk, 63);
        prev_pos63 = (uint32_t)__builtin_amdgcn_readlane((int)pp, 63);
        prev_child63 = __builtin_amdgcn_readlane(child, 63);
    }
    if (__ballot(bad) != 0ull) return false;
    kmin = wave_min_u32(kmin);
    kmax = wave_max_u32(kmax);

    // ---- 4. stable radix sort by key (descending score), only over the bits that differ ----
    const uint32_t diff = kmin ^ kmax;
    const int nbits = diff == 0u ? 0 : 32 - __clz((int)diff);
    uint32_t *srcK = keyA, *srcP = payA, *dstK = keyB, *dstP = payB;
    for (int sh = 0; sh < nbits; sh += 8) {
        wave_sync_memory();
#pragma unroll
        for (int t = 0; t < 4; t++) lds.hist[lane * 4 + t] = 0;
        wave_sync_memory();
        for (int q = lane; q < m; q += kWave) atomicAdd(&lds.hist[(srcK[q] >> sh) & 255u], 1);
        wave_sync_memory();
        int h0 = lds.hist[lane * 4 + 0], h1 = lds.hist[lane * 4 + 1], h2 = lds.hist[lane * 4 + 2],
            h3 = lds.hist[lane * 4 + 3];
        int lsum = h0 + h1 + h2 + h3;
        int excl = wave_inclusive_sum(lsum, lane) - lsum;
        wave_sync_memory();
        lds.hist[lane * 4 + 0] = excl;
        lds.hist[lane * 4 + 1] = excl + h0;
        lds.hist[lane * 4 + 2] = excl + h0 + h1;
        lds.hist[lane * 4 + 3] = excl + h0 + h1 + h2;
        wave_sync_memory();
        for (int base = 0; base < m; base += kWave) {
            const int q = base + lane;
            const bool in = q < m;
            uint32_t kk = in ? srcK[q] : 0u;
            uint32_t pay = in ? srcP[q] : 0u;
            uint32_t d = (kk >> sh) & 255u;
            // lanes of this chunk with the same digit
            uint64_t same = __ballot(in);
#pragma unroll
            for (int b = 0; b < 8; b++) {
                uint64_t bal = __ballot(in && ((d >> b) & 1u));
                same &= ((d >> b) & 1u) ? bal : ~bal;
            }
            int rank = __popcll(same & ((1ull << lane) - 1ull));
            int count = __popcll(same);
            int basepos = in ? lds.hist[d] : 0;
            if (in) {
                dstK[basepos + rank] = kk;
                dstP[basepos + rank] = pay;
            }
            wave_sync_memory();
            if (in && rank == 0) lds.hist[d] = basepos + count;
            wave_sync_memory();
        }
        uint32_t *tk = srcK;
        srcK = dstK;
        dstK = tk;
        uint32_t *tp = srcP;
        srcP = dstP;
        dstP = tp;
    }
    wave_sync_memory();

    // ---- 5. winner order: check ties across children and the last taken entry, emit ----
    uint32_t pk63 = 0u, ppay63 = 0u;
    bool have_prev = false;
    for (int base = 0; base < m; base += kWave) {
        const int q = base + lane;
        const bool in = q < m;
        uint32_t kk = in ? srcK[q] : 0u;
        uint32_t pay = in ? srcP[q] : 0u;
        uint32_t pk = (uint32_t)__shfl_up((int)kk, 1, kWave);
        uint32_t ppay = (uint32_t)__shfl_up((int)pay, 1, kWave);
        bool hp = lane > 0 || have_prev;
        if (lane == 0) {
            pk = pk63;
            ppay = ppay63;
        }
        if (in) {
            const int child = (int)((pay >> 21) & 1023u);
            const int j = (int)(pay & 0x1FFFFFu);
            a.sc_child[off + q] = child;
            a.sc_occ[off + q] = j;
            if (hp) {
                if (pk > kk) bad = true;  // not sorted
                if (pk == kk) {
                    const uint32_t pchild = (ppay >> 21) & 1023u;
                    const uint32_t ppos_ = pchild + ((ppay >> 31) ? (uint32_t)F : 0u);
                    const uint32_t pos_ = (uint32_t)child + ((pay >> 31) ? (uint32_t)F : 0u);
                    if (pchild != (uint32_t)child && ppos_ > pos_) bad = true;
                }
            }
        }
        pk63 = (uint32_t)__builtin_amdgcn_readlane((int)kk, 63);
        ppay63 = (uint32_t)__builtin_amdgcn_readlane((int)pay, 63);
        have_prev = true;
    }
    {
        // the last taken entry must come before every other child's first untaken entry
        // (its own child's next entry was checked in step 3)
        const uint32_t lk = ~srcK[m - 1];
        const uint32_t lpay = srcP[m - 1];
        const uint32_t lchild = (lpay >> 21) & 1023u;
        const uint32_t lpos = lchild + ((lpay >> 31) ? (uint32_t)F : 0u);
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (uk[r] != 0u && (uint32_t)(r * kWave + lane) != lchild && !comes_before(lk, lpos, uk[r], upos[r]))
                bad = true;
        }
    }
    if (__ballot(bad) != 0ull) return false;
#pragma unroll
    for (int r = 0; r < R; r++) cnt[r] = cv[r];
    return true;
}

// The commonest crowded node: one child wins every time.  That is the case exactly when
// the score it shows to the last visitor still comes before the first score of every
// other child and its own scores never increase on the way; both are checked on the exact
// values (m evaluations spread over the lanes).  Returns false when it is not that case.
template <int R, bool RAVE>
__device__ __forceinline__ bool single_run(const SelectArgs &a, const NodeCtx &c, int lane, const Kids<R, RAVE> &k,
                                           uint32_t bk, uint32_t bpos, int off, int m, int (&cnt)[R]) {
    constexpr int F = R * kWave;
    const uint32_t uvl = (uint32_t)a.vl;
    uint32_t hi_key, hi_pos;
    wave_best(bk, bpos, hi_key, hi_pos);
    if (hi_key == 0u) return false;
    const int best = (int)(hi_pos >= (uint32_t)F ? hi_pos - (uint32_t)F : hi_pos);
    // statistics of the best child, wave-uniform
    int tn = 0, tvl = 0, trn = 0;
    float tw = 0.0f, tp = 0.0f, trw = 0.0f;
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (r == (best >> 6)) {
            tn = k.n[r];
            tw = k.w[r];
            tp = k.p[r];
            tvl = k.vl[r];
            trn = k.rn[r];
            trw = k.rw[r];
        }
    }
    const int bl = best & 63;
    const int bn = __builtin_amdgcn_readlane(tn, bl);
    const float bw = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tw), bl));
    const float bp = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tp), bl));
    const int bvl = __builtin_amdgcn_readlane(tvl, bl);
    const int brn = __builtin_amdgcn_readlane(trn, bl);
    const float brw = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(trw), bl));
    // best first candidate of all other children
    uint32_t ok = 0u, opos = 0xFFFFFFFFu;
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (r * kWave + lane != best && k.k1[r] > ok) { ok = k.k1[r]; opos = (uint32_t)(r * kWave + lane); }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (r * kWave + lane != best && k.k2[r] > ok) { ok = k.k2[r]; opos = (uint32_t)(F + r * kWave + lane); }
    }
    uint32_t sk, spos;
    wave_best(ok, opos, sk, spos);
    // the last visitor's entry decides; then every entry is checked
    uint32_t lk, lp;
    entry_key<R, RAVE>(bn, bw, bp, bvl, brn, brw, c.ep, a.rave_k, uvl, m - 1, best, lk, lp);
    if (lk == 0u || (sk != 0u && !comes_before(lk, lp, sk, spos))) return false;
    bool bad = false;
    uint32_t carry_k = 0xFFFFFFFFu, carry_p = 0u;  // entry before the chunk
    for (int base = 0; base < m; base += kWave) {
        const int j = base + lane;
        uint32_t kk = 0u, pp = 0xFFFFFFFFu;
        if (j < m) entry_key<R, RAVE>(bn, bw, bp, bvl, brn, brw, c.ep, a.rave_k, uvl, j, best, kk, pp);
        uint32_t pk = (uint32_t)__shfl_up((int)kk, 1, kWave);
        uint32_t ppos = (uint32_t)__shfl_up((int)pp, 1, kWave);
        if (lane == 0) {
            pk = carry_k;
            ppos = carry_p;
        }
        if (j < m && (kk == 0u || comes_before(kk, pp, pk, ppos))) bad = true;
        carry_k = (uint32_t)__builtin_amdgcn_readlane((int)kk, 63);
        carry_p = (uint32_t)__builtin_amdgcn_readlane((int)pp, 63);
    }
    if (__ballot(bad) != 0ull) return false;
    for (int j = lane; j < m; j += kWave) {
        a.sc_child[off + j] = best;
        a.sc_occ[off + j] = j;
    }
    if (lane == bl) {
#pragma unroll
        for (int r = 0; r < R; r++)
            if (r == (best >> 6)) cnt[r] = m;
    }
    return true;
}

// Where the walk goes on after a multi-visitor node whose visitors all chose one child.
struct Continuation {
    int node;
    int off;
    int m;
    int np;
};

// All visitors of a multi-visitor item.  Records the chosen child of every visitor, bumps
// virtual loss, partitions the visitors by child into seg_out, writes the next path
// entry, appends one item per visited child to the next level's queue (none when all
// visitors chose the same child: then the caller walks on with them).  Returns false when
// no child takes part in the selection.
template <int R, bool RAVE>
__device__ __forceinline__ bool select_group(const ForestDev &f, const SelectArgs &a, const NodeCtx &c, int lane,
                                             const int32_t *seg_in, int32_t *seg_out, int off, int m, int depth,
                                             WaveLds<R> &lds, Continuation &next) {
    Kids<R, RAVE> k;
    int cnt[R];
    load_kids<R, RAVE>(f, c.cb, c.nelig, lane, k);
#pragma unroll
    for (int r = 0; r < R; r++) {
        score_round<R, RAVE>(k, r, c.ep, a.rave_k);
        cnt[r] = 0;
    }
    uint32_t bk, bpos;
    lane_best<R, RAVE>(k, lane, bk, bpos);
    const uint32_t uvl = a.vl > 0 ? (uint32_t)a.vl : 0u;

    bool settled = false;
    int st_replay = 0;
    if (m >= kRunMin && a.vl > 0) settled = single_run<R, RAVE>(a, c, lane, k, bk, bpos, off, m, cnt);
    if (!settled && m >= kWaterLevelMin && a.vl > 0) {
        settled = water_level<R, RAVE>(a, c, lane, k, bk, bpos, off, m, lds, cnt);
        if (!settled) st_replay = 1;
    }
    if (!settled) {
        // one visitor after the other
        for (int done = 0; done < m; done++) {
            int i = wave_pick<R, RAVE>(k, lane, bk, bpos);
            if (i < 0) return false;  // no child takes part: uniform, and then for every visitor
            if (a.vl <= 0) {
                // no virtual loss: nothing changes between visitors, they all follow the first
                for (int j = lane; j < m; j += kWave) {
                    a.sc_child[off + j] = i;
                    a.sc_occ[off + j] = j;
                }
                if (lane == (i & 63)) {
#pragma unroll
                    for (int r = 0; r < R; r++)
                        if (r == (i >> 6)) cnt[r] = m;
                }
                break;
            }
            if (lane == (i & 63)) {
                int occ = 0;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    if (r == (i >> 6)) {
                        occ = cnt[r];
                        cnt[r] = occ + 1;
                        k.vl[r] = (int)((uint32_t)k.vl[r] + uvl);
                        score_round<R, RAVE>(k, r, c.ep, a.rave_k);
                    }
                }
                lane_best<R, RAVE>(k, lane, bk, bpos);
                a.sc_child[off + done] = i;
                a.sc_occ[off + done] = occ;
            }
        }
    }
    if (a.stats && lane == 0) {
        atomicAdd(a.stats + 0, 1);
        atomicAdd(a.stats + 1, settled ? 1 : 0);
        atomicAdd(a.stats + 2, settled ? m : 0);
        atomicAdd(a.stats + 3, settled ? 0 : m);
        atomicAdd(a.stats + 4, st_replay);
    }

    // a group that stays together is walked on by this wavefront
    uint32_t lmax = 0u;
#pragma unroll
    for (int r = 0; r < R; r++) lmax = umax32(lmax, (uint32_t)cnt[r]);
    const uint32_t gmax = wave_max_u32(lmax);
    uint32_t lidx = 0xFFFFFFFFu;
#pragma unroll
    for (int r = R - 1; r >= 0; r--)
        if ((uint32_t)cnt[r] == gmax) lidx = (uint32_t)(r * kWave + lane);
    const int keep = gmax == (uint32_t)m ? (int)wave_min_u32(lidx) : -1;

    // exclusive prefix of the visit counts in child order -> segment of every child
    int carry = 0;
    int keep_np = 0;
#pragma unroll
    for (int r = 0; r < R; r++) {
        int inc = wave_inclusive_sum(cnt[r], lane);
        int excl = carry + inc - cnt[r];
        int i = r * kWave + lane;
        lds.offs[i] = excl;
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
    wave_sync_memory();
    int *path_next = a.paths + (size_t)(depth + 1) * a.stride;
    for (int j = lane; j < m; j += kWave) {
        int t = seg_in[off + j];
        int i = a.sc_child[off + j];
        path_next[t] = c.cb + i;
        seg_out[off + lds.offs[i] + a.sc_occ[off + j]] = t;
    }
    next.node = -1;
    if (keep >= 0) {
        next.node = c.cb + keep;
        next.off = off + lds.offs[keep];
        next.m = (int)gmax;
        next.np = __builtin_amdgcn_readlane(keep_np, keep & 63);
    }
    // the next step of the walk reads seg_out and reuses the LDS scratch
    wave_sync_memory();
    return true;
}

template <int RMAX, bool RAVE>
__global__ __launch_bounds__(256) void k_select_level(ForestDev f, SelectArgs a, int level) {
    __shared__ WaveLds<RMAX> s_lds[4];
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

    // walk with a group of visitors while it stays together
    while (m > 1) {
        const int32_t *seg_in = depth == 0 ? a.seg0 : a.seg[(depth - 1) & 1];
        int32_t *seg_out = a.seg[depth & 1];
        NodeCtx c = node_ctx(f, a, node, np);
        bool descended = false;
        Continuation next;
        next.node = -1;
        if (c.cc > 0 && depth < a.max_depth) {
            if (c.cc <= kWave)
                descended = select_group<1, RAVE>(f, a, c, lane, seg_in, seg_out, off, m, depth,
                                                  reinterpret_cast<WaveLds<1> &>(s_lds[wib]), next);
            else
                descended = select_group<RMAX, RAVE>(f, a, c, lane, seg_in, seg_out, off, m, depth, s_lds[wib], next);
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
