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
// partitioned by chosen child (stable, so still in traversal order): the wavefront walks on
// itself with the largest part, the other parts with several visitors become new items, and
// lone visitors go to the single-visitor walk.
//
// Which child each visitor chooses:
//  * one winner: if the best child's score for the LAST visitor still beats every other
//    child's first score and its own scores never increase, every visitor takes it.
//  * few visitors: they are played one after another on register-resident statistics --
//    score, DPP arg-max with lowest-index tie-break, bump the chosen child's virtual loss,
//    next visitor.  That is the serial order itself.
//  * many visitors ("water level"): the score child i shows to its j-th visitor of this
//    batch depends on nothing but j.  If every child's scores do not increase with j, the
//    serial winner sequence is the merge of these descending lists, i.e. the m best
//    entries (i, j) in the order (score descending, candidate position ascending, j
//    ascending).  In batches of up to 2048 entries: a search on the score threshold finds
//    how many entries each child contributes (estimated by the closed-form inverse of the
//    score, then counted exactly), the entries are evaluated in parallel into LDS, a stable
//    radix sort puts them in winner order.  Nothing is assumed: afterwards the wavefront
//    checks, on the exact binary32 values, (i) that every child's taken entries and its
//    first untaken entry do not increase and (ii) that the last taken entry still comes
//    before every child's first untaken one.  Under (i) and (ii) the serial loop provably
//    produces exactly this sequence; if either fails the node is replayed one visitor at a
//    time.  A long run of one child (its score hardly moves with virtual loss) is emitted
//    without sorting.
//  * a thousand visitors or more: the node is cut into slices of its winner order that
//    several wavefronts settle side by side, and the partition is shared out the same way
//    (see select_group).
//
// Scheduling.  Two kernels.  The multi-visitor kernel is persistent: blocks of four
// wavefronts, the first of which (the owner) takes tickets of a device-side work queue,
// waits (bounded) until the item with that number is published, and processes it; the
// other three help it through block barriers: with the batch work of larger nodes, and one of
// them shares out the visitors of a settled node (the partition) while the owner already
// walks on into the kept child.  Items depend only on their ancestors, so there is no barrier
// between tree levels: the time of a selection is the longest chain of crowded nodes.
// Settling a node needs only the NUMBER of its visitors; the list of their traversal ids is
// needed last, for the node's own partition.  The children of a heavy node are therefore
// published before their lists are written (item kind 3) and wait for a "list complete" word
// where they need it.  A visitor that is alone at a node stays alone to its leaf: blocks of
// walkers behind the teams of the same persistent launch take such visitors as the teams
// create them (one wavefront per walk, no LDS); a batch whose traversals are all alone at
// their roots is one launch of the single-visitor kernel instead.
#include <algorithm>
#include <cstddef>

#include "omk_internal.h"

namespace omk {

constexpr int kRunMin = 4;                // visitors from which the one-winner check is tried
constexpr int kWaterLevelMin = 24;        // visitors from which the parallel path is tried
constexpr int kWaterLevelMaxJ = 1 << 21;  // entries per child representable in the sort payload
constexpr int kBatchCap = 2048;           // entries put in winner order at a time (LDS resident)
constexpr int kSortBits = 8;              // widest radix digit of that sort
constexpr int kSortBins = 1 << kSortBits;
constexpr int kTeamWaves = 4;             // wavefronts per block of the multi-visitor kernel: one owner that
                                          // takes the items, three helpers for the batch work of its node
constexpr int kTeam = kTeamWaves * 64;
constexpr int kTeamMin = 96;              // batch entries from which the helpers are called in
// a batch of at most this many entries per thread is ordered by counting: a lone wavefront, the block
constexpr int kCountSortLone = 2, kCountSortTeam = 1;
constexpr int kRunShortcutMin = 128;      // entries from which a run of one child is emitted without sorting
constexpr int kScatterPart = 256;         // visitors per part of a heavy node's partition, about
constexpr int kScatterUnroll = 8;         // chunks of 64 visitors whose loads the partition issues together
constexpr int kMaxWalkerBlocks = 16;         // blocks of walkers of the persistent launch, at most
constexpr int kTeamSinglesMaxWaves = 4096;  // wavefronts up to which a batch of lone traversals is walked by blocks (one round of children per wavefront)
constexpr int kFastSinglesMax = 16384;    // traversals up to which the single-visitor kernel trades bytes for latency
constexpr int kRunShareMin = 4096;        // a node whose visitors all take one child: visitors from which the scatter
                                          // is shared out like a heavy node's instead of left to one helper

enum { kStepLeaf = 0, kStepDescended = 1, kStepParked = 2 };

// Register-resident statistics of the children a lane is responsible for: child index
// i = r * 64 + lane for round r.
template <int R, bool RAVE>
struct Kids {
    int n[R];
    float w[R];
    float p[R];
    int vl[R];
    float q2[R];  // RAVE blend of the child (second scan), constant during the selection
    uint32_t k1[R];
    uint32_t k2[R];
    bool part[R];
};

// What the owner wavefront of a block asks of its helpers; first member of the LDS scratch,
// so that it sits at the same place for every fan-out class.
enum { kOpExit = 0, kOpOrder = 1, kOpEmit = 2, kOpRun = 3, kOpPartition = 4, kOpLoad = 5, kOpChain = 6 };
struct TeamCmd {
    int op;
    int rounds;  // R of the node's fan-out class: 1, or the kernel's RMAX
    int total;   // entries of the batch
    int keep;    // of which the first `keep` are winners
    int goff;    // where the batch's winners go in sc_child / sc_occ
    int cur;     // which of the two buffers holds the ordered batch
    float ep;
    uint32_t uvl;
    // kOpRun: a run of `total` entries of child `best` from its visit btk on
    int best, btk, bn, bvl;
    float bw, bp, bq2;
    uint32_t hk, hp, sk, spos;
    int proven;  // kOpRun: the child's keys provably do not increase over the run
    // kOpPartition: the node whose visitors a helper shares out while the owner walks on
    int j_cb, j_off, j_m, j_depth, j_keep, j_run_child;
    // kOpPartition: the node the owner walks on into (-1: none) and its N_parent: the two helpers that
    // do not partition load and score their share of that node's children meanwhile (load_ahead).
    // kOpLoad: the same for the node the owner has just taken from the queue, whose child range it
    // knows (pre_cb, pre_cc; pre_cc < 0: not known, the helpers fetch it)
    int pre_node, pre_np, pre_cb, pre_cc;
    // kOpChain: the node a chain walk starts at (chain_walk), its N, child range, depth, and its visitors
    int c_node, c_np, c_cb, c_cc, c_depth, c_off, c_m;
};

// What that helper reads, at the same place for every fan-out class: the owner's next node
// uses the scratch of its own class (WaveLds) meanwhile, and leaves this alone until the
// helper is done.
template <int RMAX>
struct PartLds {
    int offs[RMAX * kWave];  // start of every child's segment in the node's visitor list
    int cnt[RMAX * kWave];   // visitors of every child
    int np[RMAX * kWave];    // visit count of every child (its children's N_parent)
    int lone[RMAX * kWave];  // rank of the child among those with one visitor
    uint32_t order[kHeavyMin];  // (child, visit number) of every visitor in winner order (ordinary nodes only)
};

// Scratch in LDS of one block of the multi-visitor kernel (one node at a time).
template <int R>
struct WaveLds {
    TeamCmd cmd;
    uint32_t red[4];       // team reductions: smallest / largest inverted key, flags
    int wsum[kTeamWaves];  // team prefix scan: totals of the wavefronts
    int offs[R * kWave];   // exclusive prefix of the visit counts in child order
    int st_n[R * kWave];   // statistics of every child, readable by any lane
    float st_w[R * kWave];
    float st_p[R * kWave];
    int st_vl[R * kWave];
    float st_q2[R * kWave];
    int st_j0[R * kWave];  // visits already settled / visit count, by phase
    int hist[kSortBins * (kBatchCap / kWave + 1) > R * kWave ? kSortBins * (kBatchCap / kWave + 1) : R * kWave];  // sort: entries per (digit value, block of 64); emit: visits per child
    uint32_t pay[R * kWave];      // per child: entries of the batch
    alignas(16) uint32_t key[2][kBatchCap];  // entries of the batch being ordered: inverted score key ...
    alignas(16) uint32_t pay2[2][kBatchCap];  // ... and pass flag, child, visit number; two buffers, ping-pong
};

// AHEAD: ask for the statistics of every child in range before the legality bits are known
// (one memory round trip instead of two; reads the statistics of illegal children too, so
// only where latency matters more than traffic).
// SPAN (with AHEAD): the child range of every child in range comes along (sp[r], like the
// statistics), so that a walk that goes on into one of them does not make one more dependent trip
// to memory for it.
template <int R, bool RAVE, bool AHEAD = false, bool SPAN = false>
__device__ __forceinline__ void load_kids(const ForestDev &f, int cb, int nelig, int lane, float rave_k,
                                          Kids<R, RAVE> &k, int2 *sp = nullptr) {
    static_assert(AHEAD || !SPAN, "the child ranges are only fetched by the look-ahead variant");
    if (AHEAD) {
        uint32_t word[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int i = r * kWave + lane;
            const bool in = i < nelig;
            const int id = cb + i;
            word[r] = in && f.legal ? f.legal[(uint32_t)id >> 5] : 0xFFFFFFFFu;
            k.n[r] = in ? f.N[id] : 0;
            k.w[r] = in ? f.W[id] : 0.0f;
            k.p[r] = in ? f.P[id] : 0.0f;
            k.vl[r] = in ? f.VL[id] : 0;
            k.q2[r] = RAVE && in ? f.q2[id] : 0.0f;  // the RAVE blend, kept per node (k_blend_all, k_blend_paths)
            if (SPAN) sp[r] = in ? f.span[id] : int2{0, 0};
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int i = r * kWave + lane;
            const int id = cb + i;
            const bool in = i < nelig && ((word[r] >> ((uint32_t)id & 31u)) & 1u);
            k.part[r] = in;
            if (!in) {
                k.n[r] = 0;
                k.w[r] = 0.0f;
                k.p[r] = 0.0f;
                k.vl[r] = 0;
                k.q2[r] = 0.0f;
            }
        }
        return;
    }
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
        k.q2[r] = RAVE && in ? f.q2[id] : 0.0f;
    }
}

template <int R, bool RAVE>
__device__ __forceinline__ void score_round(Kids<R, RAVE> &k, int r, float ep) {
    uint32_t a = 0u, b = 0u;
    if (k.part[r]) child_keys<RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.q2[r], ep, a, b);
    k.k1[r] = a;
    k.k2[r] = b;
}

// Rounds R0 .. R1-1 of load_kids (look-ahead variant) and score_round; the other rounds of k are
// left alone.
template <int R, bool RAVE, int R0, int R1>
__device__ __forceinline__ void load_score_rounds(const ForestDev &f, int cb, int nelig, int lane, float rave_k,
                                                  float ep, Kids<R, RAVE> &k) {
    uint32_t word[R];
#pragma unroll
    for (int r = R0; r < R1; r++) {
        const int i = r * kWave + lane;
        const bool in = i < nelig;
        const int id = cb + i;
        word[r] = in && f.legal ? f.legal[(uint32_t)id >> 5] : 0xFFFFFFFFu;
        k.n[r] = in ? f.N[id] : 0;
        k.w[r] = in ? f.W[id] : 0.0f;
        k.p[r] = in ? f.P[id] : 0.0f;
        k.vl[r] = in ? f.VL[id] : 0;
        k.q2[r] = RAVE && in ? f.q2[id] : 0.0f;
    }
#pragma unroll
    for (int r = R0; r < R1; r++) {
        const int i = r * kWave + lane;
        const int id = cb + i;
        const bool in = i < nelig && ((word[r] >> ((uint32_t)id & 31u)) & 1u);
        k.part[r] = in;
        if (!in) {
            k.n[r] = 0;
            k.w[r] = 0.0f;
            k.p[r] = 0.0f;
            k.vl[r] = 0;
            k.q2[r] = 0.0f;
        }
        score_round<R, RAVE>(k, r, ep);
    }
}

// A wide node that its owner walks on into (fan-out class R > 1) is loaded by three wavefronts of the
// block: while one helper shares out the visitors of the node before it, the owner takes the first
// kAheadShare rounds of the children and the other two helpers the rest, which they leave in LDS
// (statistics, blend, keys); the owner collects them at the barrier that ends the partition request.
// One wavefront issues an instruction every few cycles at best, and six rounds of divisions and square
// roots (two scans, RAVE blend) are a few microseconds of that on every node of the chain.
template <int R>
struct AheadShare {
    static constexpr int kRounds = (R + 2) / 3;
};

template <int R, bool RAVE>
__device__ __forceinline__ void load_ahead(const ForestDev &f, const SelectArgs &a, WaveLds<R> &lds, int node, int np,
                                           int cb, int cc, int wave, int lane);

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
    if (RAVE && m != 0u && pos >= (uint32_t)(R * kWave)) {
        // a candidate of the second scan: the reference only runs that scan when the first one
        // found a child (mcts_node.cpp:173-184); with no real first-scan score it falls back
        bool any1 = false;
#pragma unroll
        for (int r = 0; r < R; r++) any1 |= k.k1[r] != 0u;
        if (__ballot(any1) == 0ull) m = 0u;
    }
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

__device__ __forceinline__ NodeCtx node_ctx(const ForestDev &f, const SelectArgs &a, int node, int np,
                                            bool have_span = false, int2 span = int2{0, 0}) {
    NodeCtx c;
    int2 sp = have_span ? span : f.span[node];
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

template <int R, bool RAVE>
__device__ __forceinline__ void load_ahead(const ForestDev &f, const SelectArgs &a, WaveLds<R> &lds, int node, int np,
                                           int cb, int cc, int wave, int lane) {
    constexpr int S = AheadShare<R>::kRounds;
    const NodeCtx c = node_ctx(f, a, node, np, cc >= 0, int2{cb, cc});
    if (c.cc <= kWave) return;  // a leaf, or a node of the narrow class: its owner loads it alone
    Kids<R, RAVE> k;
    if (wave == 2) load_score_rounds<R, RAVE, (S < R ? S : R), (2 * S < R ? 2 * S : R)>(f, c.cb, c.nelig, lane, a.rave_k, c.ep, k);
    else load_score_rounds<R, RAVE, (2 * S < R ? 2 * S : R), R>(f, c.cb, c.nelig, lane, a.rave_k, c.ep, k);
    const int r0 = wave == 2 ? S : 2 * S, r1 = wave == 2 ? 2 * S : R;
#pragma unroll
    for (int r = S; r < R; r++) {
        if (r >= r0 && r < r1) {
            const int i = r * kWave + lane;
            lds.st_n[i] = k.n[r];
            lds.st_w[i] = k.w[r];
            lds.st_p[i] = k.p[r];
            lds.st_vl[i] = k.vl[r];
            lds.st_q2[i] = k.q2[r];
            lds.key[0][i] = k.k1[r];
            lds.key[1][i] = k.k2[r];
            lds.pay[i] = k.part[r] ? 1u : 0u;
        }
    }
}

// One selection for a single visitor.  Returns the child index or -1; np_child receives
// the visit count of the chosen child (the next node's N_parent).
//
// A walk is a chain of dependent trips to memory: child range, legality bits, statistics, three per
// level on a layout with a legal mask.  AHEAD asks for the statistics of all children in range
// before the legality bits are known (two trips; the cache lines of the illegal ones are fetched
// anyway).  FAST, for a launch with few walkers and an idle memory system, also asks for the child
// ranges of all of them (one trip, about 1.5 times the bytes); span_child then receives the chosen
// child's range.
template <int R, bool RAVE, bool AHEAD, bool FAST>
__device__ __forceinline__ int select_single(const ForestDev &f, const SelectArgs &a, const NodeCtx &c, int lane,
                                             int &np_child, int2 &span_child) {
    static_assert(AHEAD || !FAST, "FAST includes AHEAD");
    Kids<R, RAVE> k;
    int2 sp[R];
    load_kids<R, RAVE, AHEAD, FAST>(f, c.cb, c.nelig, lane, a.rave_k, k, sp);
#pragma unroll
    for (int r = 0; r < R; r++) score_round<R, RAVE>(k, r, c.ep);
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
    if (FAST) {
        int sx = 0, sy = 0;
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (r == (i >> 6)) {
                sx = sp[r].x;
                sy = sp[r].y;
            }
        }
        span_child.x = __builtin_amdgcn_readlane(sx, i & 63);
        span_child.y = __builtin_amdgcn_readlane(sy, i & 63);
    }
    return i;
}

// Key and candidate position child `child` shows to the visitor that finds its counter at
// vl0 + j * uvl.
template <int R, bool RAVE>
__device__ __forceinline__ void entry_key(int n, float w, float p, int vl0, float q2, float ep, uint32_t uvl, int j,
                                          int child, uint32_t &key, uint32_t &pos) {
    int vlj = (int)((uint32_t)vl0 + (uint32_t)j * uvl);
    uint32_t k1, k2;
    child_keys<RAVE>(n, w, p, vlj, q2, ep, k1, k2);
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

// Inverse of score_key for real keys: the score a key stands for.
__device__ __forceinline__ float key_score(uint32_t key) {
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key);
}

// ESTIMATE of how many of a child's next entries score at least tau, from the closed form
// of the score as a function of x = N + VL:  s1(x) = (W+N)/x - 1 + c/(1+x)  (c = P * ep) and,
// with RAVE, s2(x) = q2 + c/(1+x).  Fast approximate arithmetic on purpose: the result only
// seeds the exact search, which tests the two entries around it.
template <bool RAVE>
__device__ __forceinline__ int predict_count(int n, float w, float p, int vl, float q2, float ep, uint32_t uvl,
                                             float tau, int cap) {
    const float x0 = (float)n + (float)vl;
    const float A = w + (float)n;
    const float cc = p * ep;
    const float inv_step = __frcp_rn((float)uvl);
    float xs = -1.0f;  // largest x with score >= tau
    const float a2 = tau + 1.0f;
    if (a2 > 1e-12f) {
        const float b2 = a2 - A - cc;
        const float disc = b2 * b2 + 4.0f * a2 * A;
        if (disc >= 0.0f) xs = (-b2 + __fsqrt_rn(disc)) * __frcp_rn(2.0f * a2);
    } else {
        xs = 3.0e38f;
    }
    if (RAVE) {
        const float d = tau - q2;
        float x2 = d > 1e-12f ? cc * __frcp_rn(d) - 1.0f : 3.0e38f;
        xs = fmaxf(xs, x2);
    }
    float cnt = floorf((xs - x0) * inv_step) + 1.0f;
    if (!(cnt > 0.0f)) return 0;
    return cnt >= (float)cap ? cap : (int)cnt;
}

constexpr int kChainMaxLevels = 64;  // levels one walk records; a longer chain goes on as another walk

struct ChainLds {
    int levels;                  // levels walked
    int nodes[kChainMaxLevels];  // the child taken at every one of them
    int e_node, e_np, e_cb, e_cc, e_depth;  // where the walk stands: a node that has not been settled
    int e_kids;       // that node's children are in the LDS scratch (it failed the one-winner test), with:
    int e_contested;  // single_run's verdict: the best child's entry for the last visitor is real but not first,
    int e_best0;      // that child,
    uint32_t e_lk0;   // that entry's key,
    int e_second;     // and whether it is a candidate of the second scan
    int n_barriers;   // -1 while a walk is under way, then the number of block barriers it took
};
typedef __attribute__((address_space(3))) unsigned char *LdsBytesP;
// one per block of the multi-visitor kernel
__shared__ ChainLds g_chain;
// The timeline, when it is switched on: what a slice of a heavy node did (100 MHz clock): [0] thresholds and
// exact counts, [1] its batch(es), [2] entries of its first batch, or -1 when it had to search for it, [3] visitors
// it settled.  One per block.
__shared__ int g_slice_note[4];


// The owner may have left the partition of its previous node with a helper: the block
// barrier that ends that request is still open.  Everything that needs the helpers, the
// visitor lists that partition writes, or the LDS it reads, closes it first.
__device__ __forceinline__ void close_pending(bool &pending) {
    if (pending) {
        __syncthreads();
        pending = false;
    }
}

// An item of kind 3 was published before its visitor list was written (the children of a
// heavy node, whose visitors several wavefronts share out): wait for the list.  Bounded like
// every wait; false when the selection is given up.
__device__ __forceinline__ bool wait_list(const SelectArgs &a, int off, int depth, int lane) {
    bool ok = false;
    for (int spins = 0;; spins++) {
        int v = 0, ab = 0;
        if (lane == 0) {
            v = __hip_atomic_load(a.list_flag + off, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (v < depth && (spins & 3) == 3)
                ab = __hip_atomic_load(a.sched_wait + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        v = __builtin_amdgcn_readfirstlane(v);
        ab = __builtin_amdgcn_readfirstlane(ab);
        if (v >= depth) {
            ok = true;
            break;
        }
        if (ab) break;
        if (spins >= a.spin_limit) {
            if (lane == 0 && atomicCAS(a.sched_wait + 1, 0, 3) == 0) {
                a.sched_wait[2] = off;  // which list never came, for the error message
                a.sched_wait[3] = depth;
                a.sched_wait[4] = v;
            }
            break;
        }
        __builtin_amdgcn_s_sleep(8);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    return ok;
}

// A key in [lo_key, hi_key] whose estimated entry count est(key) (wave-uniform, non-increasing in
// the key) lands in the window [target, acc_hi], or failing that in [acc_below, target); the largest
// key found with est >= target otherwise.  est(lo_key) >= target and est(hi_key) < target are taken
// for granted.  The count is close to a hyperbola in the score, alpha / (score + 1) - beta (every
// child's next visits score about (W + N + c) / x - 1), so the search works in y = 1 / (score + 1),
// where the count is nearly a straight line: false position between the ends of its bracket, with
// the value of an end that stays put halved at every step that leaves it there (the Illinois rule:
// the ends' counts are capped per child and would otherwise pin the interpolation), the first
// step from made-up end values.  Halving the KEY interval instead takes a dozen steps whenever the
// bracket straddles score zero, where the keys are densest.  Deterministic: the same arguments
// give the same key on every wavefront.  Only efficiency depends on the result: whatever key comes
// out, the caller counts exactly.
// plateau(klo, khi), asked now and then once six steps have not brought the count into the window: a key
// to return at once, or 0.
template <typename Est, typename Plateau>
__device__ __forceinline__ uint32_t search_threshold(uint32_t lo_key, uint32_t hi_key, int target, int acc_hi,
                                                     int acc_below, int &evals, Est est, Plateau plateau) {
    uint32_t klo = lo_key, khi = hi_key;
    auto y_of = [](uint32_t k) {
        float d = key_score(k) + 1.0f;
        d = d > 1e-6f ? d : 1e-6f;
        return __frcp_rn(d);
    };
    float ylo = y_of(klo), yhi = y_of(khi);
    const float aim = (float)target + 0.5f * (float)(acc_hi - target);
    float flo = aim, fhi = -aim;  // count minus aim at the two ends: made up until an end has been evaluated
    int last = 0;                 // which end the last step moved: +1 the low one, -1 the high one
    for (int it = 0; it < 48 && khi - klo > 1u; it++) {
        const float ym = (ylo * fhi - yhi * flo) * __frcp_rn(fhi - flo);
        uint32_t kmid = score_key(__frcp_rn(ym) - 1.0f);
        if (!(kmid > klo)) kmid = klo + 1u;
        if (!(kmid < khi)) kmid = khi - 1u;
        // the dense sliver: once false position stops moving off an end, halve the key interval
        if (it >= 12) kmid = klo + ((khi - klo) >> 1);
        const int e = est(kmid);
        evals++;
        if (e >= target) {
            klo = kmid;
            ylo = y_of(kmid);
            flo = (float)e - aim;
            if (e <= acc_hi) break;
            if (last > 0) fhi *= 0.5f;
            last = 1;
        } else {
            if (e >= acc_below) {
                klo = kmid;
                break;
            }
            khi = kmid;
            yhi = y_of(kmid);
            fhi = (float)e - aim;
            if (last < 0) flo *= 0.5f;
            last = -1;
        }
        if (it >= 5 && (it - 5) % 3 == 0 && it <= 17 && khi - klo > 1u) {
            const uint32_t kp = plateau(klo, khi);
            if (kp >= lo_key && kp <= hi_key && kp != 0u) return kp;
        }
    }
    return klo;
}

template <typename Est>
__device__ __forceinline__ uint32_t search_threshold(uint32_t lo_key, uint32_t hi_key, int target, int acc_hi,
                                                     int acc_below, int &evals, Est est) {
    return search_threshold(lo_key, hi_key, target, acc_hi, acc_below, evals, est,
                            [](uint32_t, uint32_t) { return 0u; });
}

template <int NT>
__device__ __forceinline__ void team_sync() {
    if (NT == kWave) wave_sync_memory();
    else __syncthreads();
}

// One batch of a crowded node, steps 2 and 3: evaluate its entries in (child, visit) order
// into LDS (child i contributes pay[i] entries starting at offs[i], from visit st_j0[i] on),
// then put them in winner order.  Run by NT threads with the same arguments: one wavefront,
// or the whole block (the owner wavefront and its helpers).  Returns which buffer holds the
// ordered batch; red[2] bit 2 is set when an entry has no real key or a child's entries
// increase.
template <int R, bool RAVE, int NT>
__device__ __forceinline__ int batch_order(WaveLds<R> &lds, int tid, int total, float ep, uint32_t uvl) {
    constexpr int F = R * kWave;
    const int lane = tid & 63;
    if (tid == 0) {
        lds.red[0] = 0xFFFFFFFFu;
        lds.red[1] = 0u;
        lds.red[2] = 0u;
    }
    team_sync<NT>();
    // every thread evaluates a contiguous run of `per` entries (odd, so that the LDS writes of
    // the threads fall into different banks)
    const int per = ((total + NT - 1) / NT) | 1;
    const int q0 = tid * per < total ? tid * per : total;
    const int q1 = q0 + per < total ? q0 + per : total;
    {
        bool bad_entry = false;
        bool kind1 = false, kind2 = false;  // candidates of the first / second scan present
        uint32_t kmin = 0xFFFFFFFFu, kmax = 0u;
        int q = q0;
        int child = 0, seg_end = 0;
        int sn = 0, svl = 0, sj0 = 0;
        float sw = 0.0f, sp = 0.0f, sq2 = 0.0f;
        uint32_t pk = 0u, ppos = 0u;
        bool have = false;
        if (q < q1) {
            // last child whose segment starts at or before q
            int lo_i = 0, hi_i = F;
            while (hi_i - lo_i > 1) {
                int mid = (lo_i + hi_i) >> 1;
                if (lds.offs[mid] <= q) lo_i = mid;
                else hi_i = mid;
            }
            child = lo_i;
            seg_end = lds.offs[child] + (int)lds.pay[child];
        }
        bool fresh = true;
        uint32_t firstk = 0u, firstp = 0u;
        int firstj = 0;
        for (; q < q1; q++) {
            while (q >= seg_end) {  // next child with entries
                child++;
                seg_end = lds.offs[child] + (int)lds.pay[child];
                fresh = true;
            }
            if (fresh) {
                sn = lds.st_n[child];
                sw = lds.st_w[child];
                sp = lds.st_p[child];
                svl = lds.st_vl[child];
                sq2 = lds.st_q2[child];
                sj0 = lds.st_j0[child];
                fresh = false;
                have = false;
            }
            const int jl = q - lds.offs[child];
            uint32_t kk, pp;
            entry_key<R, RAVE>(sn, sw, sp, svl, sq2, ep, uvl, jl, child, kk, pp);
            lds.key[0][q] = ~kk;
            lds.pay2[0][q] = (pp >= (uint32_t)F ? 0x80000000u : 0u) | ((uint32_t)child << 21) | (uint32_t)(sj0 + jl);
            kmin = umin32(kmin, ~kk);
            kmax = umax32(kmax, ~kk);
            if (pp >= (uint32_t)F) kind2 = true;
            else kind1 = true;
            if (kk == 0u) bad_entry = true;
            // within a child the entries must not increase
            if (have && comes_before(kk, pp, pk, ppos)) bad_entry = true;
            if (q == q0) {
                firstk = kk;
                firstp = pp;
                firstj = jl;
            }
            pk = kk;
            ppos = pp;
            have = true;
        }
        kmin = wave_min_u32(kmin);
        kmax = wave_max_u32(kmax);
        const uint32_t flags = (__ballot(kind1) != 0ull ? 1u : 0u) | (__ballot(kind2) != 0ull ? 2u : 0u) |
                               (__ballot(bad_entry) != 0ull ? 4u : 0u);
        if (lane == 0) {
            atomicMin(&lds.red[0], kmin);
            atomicMax(&lds.red[1], kmax);
            atomicOr(&lds.red[2], flags);
        }
        // a small batch is ordered by counting (below), four entries per LDS read: keys behind
        // its last entry that never count
        if (total <= (NT == kWave ? kCountSortLone : kCountSortTeam) * NT && tid < 4)
            lds.key[0][total + tid] = 0xFFFFFFFFu;
        team_sync<NT>();
        // the run of the previous thread may end inside the same child: check the seam
        bool bad_seam = false;
        if (q0 < q1 && firstj > 0) {
            const uint32_t lk = ~lds.key[0][q0 - 1];
            const uint32_t lpay = lds.pay2[0][q0 - 1];
            const uint32_t lp = ((lpay >> 21) & 1023u) + ((lpay >> 31) ? (uint32_t)F : 0u);
            if (comes_before(firstk, firstp, lk, lp)) bad_seam = true;
        }
        if (__ballot(bad_seam) != 0ull && lane == 0) atomicOr(&lds.red[2], 4u);
    }
    // the same for every thread: keep them on the scalar unit, the loops below hold barriers
    const uint32_t kmin = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds.red[0]);
    const uint32_t kmax = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds.red[1]);
    const bool mixed = ((uint32_t)__builtin_amdgcn_readfirstlane((int)lds.red[2]) & 3u) == 3u;

    // A small batch (at most kCountSortLone / kCountSortTeam entries per thread): the rank of an
    // entry is the number of entries that come before it, counted against every entry of the
    // batch (one 16-byte LDS read serves four of them, the same address for all lanes).  Same
    // order as the radix sort below: inverted key ascending, then scan kind, child and visit
    // number, which is the payload as a number: key and payload are compared as one 64-bit
    // number (children tied on a key are common, so the payload is not left to a second pass).
    constexpr int kCountSortPerThread = NT == kWave ? kCountSortLone : kCountSortTeam;
    if (total <= kCountSortPerThread * NT) {
        const uint32_t *src_k = lds.key[0], *src_p = lds.pay2[0];
        uint32_t mk[kCountSortPerThread], mp[kCountSortPerThread];
        uint64_t mine[kCountSortPerThread];
        int rk[kCountSortPerThread];
#pragma unroll
        for (int e = 0; e < kCountSortPerThread; e++) {
            const int q = tid + e * NT;
            mk[e] = q < total ? src_k[q] : 0xFFFFFFFFu;
            mp[e] = q < total ? src_p[q] : 0xFFFFFFFFu;
            mine[e] = ((uint64_t)mk[e] << 32) | mp[e];
            rk[e] = 0;
        }
#pragma unroll 4
        for (int q4 = 0; q4 < total; q4 += 4) {
            const uint4 ok = *reinterpret_cast<const uint4 *>(src_k + q4);
            const uint4 op = *reinterpret_cast<const uint4 *>(src_p + q4);
            const uint64_t o0 = ((uint64_t)ok.x << 32) | op.x, o1 = ((uint64_t)ok.y << 32) | op.y;
            const uint64_t o2 = ((uint64_t)ok.z << 32) | op.z, o3 = ((uint64_t)ok.w << 32) | op.w;
#pragma unroll
            for (int e = 0; e < kCountSortPerThread; e++)
                rk[e] += (int)(o0 < mine[e]) + (int)(o1 < mine[e]) + (int)(o2 < mine[e]) + (int)(o3 < mine[e]);
        }
#pragma unroll
        for (int e = 0; e < kCountSortPerThread; e++) {
            if (tid + e * NT < total) {
                lds.key[1][rk[e]] = mk[e];
                lds.pay2[1][rk[e]] = mp[e];
            }
        }
        team_sync<NT>();
        return 1;
    }

    // Stable radix sort, in LDS.  Order wanted: key descending, then candidate position
    // ascending, then visit number.  The entries start in (child, visit) order; least
    // significant digit first: a one-bit pass on the scan kind (only when both kinds occur:
    // candidates of the first scan sit before those of the second), then the bits of the key
    // range in digits of up to kSortBits bits.  One pass: the current order is cut in blocks
    // of 64 entries, one per lane of a wavefront; inside a block every lane finds the lanes
    // that hold the same digit value (one ballot per bit), which gives its rank among them
    // and their number; the numbers go to a table indexed (digit value, block), an
    // exclusive scan over the table in that order gives every (value, block) group its start,
    // and every lane moves its entry to start + rank: stable.
    const uint32_t range = kmax - kmin;
    const int nbits = range == 0u ? 0 : 32 - __clz((int)range);
    constexpr int kWaves = NT / kWave;
    constexpr int kRounds = NT == kWave ? 4 : kBatchCap / NT;  // blocks a wavefront can be given
    static_assert(kTeamMin <= 4 * kWave, "a lone wavefront orders fewer than four blocks");
    const int wave = tid >> 6;
    const int nblocks = (total + kWave - 1) >> 6;
    const int nb1 = nblocks | 1;  // odd table stride: the lanes of a wavefront hit different LDS banks
    int cur = 0;
    const int key_passes = (nbits + kSortBits - 1) / kSortBits;
    const int bits_even = key_passes > 0 ? (nbits + key_passes - 1) / key_passes : 0;
    for (int pass = mixed ? -1 : 0; pass < key_passes; pass++) {
        const int sh = pass * bits_even;
        const int bits = pass < 0 ? 1 : (nbits - sh < bits_even ? nbits - sh : bits_even);
        const int ndig = 1 << bits;
        const uint32_t *src_k = lds.key[cur], *src_p = lds.pay2[cur];
        uint32_t *dst_k = lds.key[cur ^ 1], *dst_p = lds.pay2[cur ^ 1];
        uint32_t kk[kRounds], pp[kRounds];
        int dig[kRounds], rank[kRounds];
#pragma unroll
        for (int r = 0; r < kRounds; r++) {
            const int blk = wave + r * kWaves;
            if (blk < nblocks) {  // uniform per wavefront
                const int q = blk * kWave + lane;
                const bool valid = q < total;
                kk[r] = valid ? src_k[q] : 0u;
                pp[r] = valid ? src_p[q] : 0u;
                const uint32_t d = pass < 0 ? pp[r] >> 31 : ((kk[r] - kmin) >> sh) & (uint32_t)(ndig - 1);
                uint64_t same = __ballot(valid);
                for (int bb = 0; bb < bits; bb++) {
                    const bool one = (d >> bb) & 1u;
                    const uint64_t bal = __ballot(one);
                    same &= one ? bal : ~bal;
                }
                dig[r] = (int)d;
                rank[r] = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(same >> 32),
                                                         __builtin_amdgcn_mbcnt_lo((uint32_t)same, 0u));
                for (int dv = lane; dv < ndig; dv += kWave) {
                    lds.hist[dv * nb1 + blk] = 0;
                    if (blk == 0 && nb1 != nblocks) lds.hist[dv * nb1 + nblocks] = 0;  // the pad column
                }
                wave_sync_memory();
                if (valid && rank[r] == 0) lds.hist[(int)d * nb1 + blk] = __popcll(same);
            }
        }
        team_sync<NT>();
        {
            // exclusive scan of the table: every thread owns `own` consecutive counters
            const int n_tab = ndig * nb1;
            const int own = (n_tab + NT - 1) / NT;
            const int t0 = tid * own < n_tab ? tid * own : n_tab;
            const int t1 = t0 + own < n_tab ? t0 + own : n_tab;
            int lsum = 0;
            for (int t = t0; t < t1; t++) lsum += lds.hist[t];
            const int inc = wave_inclusive_sum(lsum, lane);
            int run = inc - lsum;
            if (NT > kWave) {
                if (lane == kWave - 1) lds.wsum[wave] = inc;
                team_sync<NT>();
                for (int w = 0; w < wave; w++) run += lds.wsum[w];
            }
            for (int t = t0; t < t1; t++) {
                const int h = lds.hist[t];
                lds.hist[t] = run;
                run += h;
            }
        }
        team_sync<NT>();
#pragma unroll
        for (int r = 0; r < kRounds; r++) {
            const int blk = wave + r * kWaves;
            if (blk < nblocks && blk * kWave + lane < total) {
                const int pos = lds.hist[dig[r] * nb1 + blk] + rank[r];
                dst_k[pos] = kk[r];
                dst_p[pos] = pp[r];
            }
        }
        team_sync<NT>();
        cur ^= 1;
    }
    team_sync<NT>();
    return cur;
}

// Step 4 of a batch: the first `keep` entries of the ordered batch are the next winners;
// records (child, visit number) of each at its rank, leaves in hist[i] the visits child i
// has after them, and checks the order of the whole batch, kept or not (what is dropped
// must come after what is kept): red[2] bit 2 on failure.
template <int R, int NT>
__device__ __forceinline__ void batch_emit(const SelectArgs &a, WaveLds<R> &lds, uint32_t *order, int tid, int total,
                                           int keep, int goff, int cur) {
    constexpr int F = R * kWave;
    const uint32_t *skey = lds.key[cur], *spay = lds.pay2[cur];
    for (int i = tid; i < F; i += NT) lds.hist[i] = 0;
    team_sync<NT>();
    bool bad_order = false;
    for (int q = tid; q < total; q += NT) {
        const uint32_t kk = skey[q];
        const uint32_t pay = spay[q];
        const int child = (int)((pay >> 21) & 1023u);
        const int j = (int)(pay & 0x1FFFFFu);
        if (q < keep) {
            if (goff >= 0) {
                a.sc_child[goff + q] = child;
                a.sc_occ[goff + q] = j;
            } else {  // the node's only batch: the partition reads the order from LDS
                order[q] = pay;
            }
            atomicMax(&lds.hist[child], j + 1);
        }
        if (q > 0) {
            const uint32_t pk = skey[q - 1];
            const uint32_t ppay = spay[q - 1];
            if (pk > kk) bad_order = true;  // not sorted
            if (pk == kk) {
                const uint32_t pchild = (ppay >> 21) & 1023u;
                const uint32_t ppos_ = pchild + ((ppay >> 31) ? (uint32_t)F : 0u);
                const uint32_t pos_ = (uint32_t)child + ((pay >> 31) ? (uint32_t)F : 0u);
                if (pchild != (uint32_t)child && ppos_ > pos_) bad_order = true;
            }
        }
    }
    if (__ballot(bad_order) != 0ull && (tid & 63) == 0) atomicOr(&lds.red[2], 4u);
    team_sync<NT>();
}

// A run of L entries of one child (visits btk .. btk + L - 1), about to be emitted as the
// next L winners at ranks goff ..: every entry must have a real key and must not come before
// its predecessor (the first one's predecessor is the child's current head (hk, hp), i.e.
// itself), and the last one must still come before the others' best (sk, spos).  The
// entries are written whether or not the checks hold; red[2] bit 2 reports a failure.
// proven: the child's keys provably do not increase over these visits (keys_provably_monotone), so
// only the run's last entry is evaluated.
template <int R, bool RAVE, int NT>
__device__ __forceinline__ void batch_run(const SelectArgs &a, WaveLds<R> &lds, int tid, int L, int goff, int best,
                                          int btk, int bn, float bw, float bp, int bvl, float bq2, float ep,
                                          uint32_t uvl, uint32_t hk, uint32_t hp, uint32_t sk, uint32_t spos,
                                          bool proven) {
    const int per = (L + NT - 1) / NT;
    const int j0 = tid * per < L ? tid * per : L;
    const int j1 = j0 + per < L ? j0 + per : L;
    bool bad_run = false;
    if (proven) {
        if (tid == 0) {
            uint32_t kk, p2;
            entry_key<R, RAVE>(bn, bw, bp, bvl, bq2, ep, uvl, btk + L - 1, best, kk, p2);
            if (kk == 0u || hk == 0u || (sk != 0u && !comes_before(kk, p2, sk, spos))) bad_run = true;
        }
    } else if (j0 < j1) {
        uint32_t pk = hk, pp = hp;
        if (j0 > 0) entry_key<R, RAVE>(bn, bw, bp, bvl, bq2, ep, uvl, btk + j0 - 1, best, pk, pp);
        for (int j = j0; j < j1; j++) {
            uint32_t kk, p2;
            entry_key<R, RAVE>(bn, bw, bp, bvl, bq2, ep, uvl, btk + j, best, kk, p2);
            if (kk == 0u || comes_before(kk, p2, pk, pp)) bad_run = true;
            if (j == L - 1 && sk != 0u && !comes_before(kk, p2, sk, spos)) bad_run = true;
            pk = kk;
            pp = p2;
        }
    }
    for (int j = tid; j < L; j += NT) {
        a.sc_child[goff + j] = best;
        a.sc_occ[goff + j] = btk + j;
    }
    if (__ballot(bad_run) != 0ull && (tid & 63) == 0) atomicOr(&lds.red[2], 4u);
    team_sync<NT>();
}

// The children of a node that can contribute entries at or above a lower bound, listed
// densely (one per lane and round) so that work on them costs one round per 64 ACTIVE
// children instead of one per 64 children.
template <int R>
struct ActiveSet {
    int rounds;
    int c[R];  // child index, -1 = none
    int n[R];
    int vl[R];
    float w[R], p[R], q2[R];
    uint32_t head[R];
};

// Exact number of entries of every active child at or above threshold T (at most m each):
// the closed-form estimate, then the two entries around it are tested with the exact
// arithmetic; if the estimate is further off, gallop away from it and bisect the rest.
// A child whose key hardly moves with virtual loss (a RAVE blend that dominates) defeats the
// estimate by thousands of entries at a threshold near its plateau: a few such children
// left after three gallop steps are counted by the whole wavefront instead, one child at a
// time, 64 candidate counts per round (two or three rounds where the lane alone takes
// twenty-odd evaluations while the other 63 wait).
constexpr int kCoopCountMax = 4;  // children counted that way per round of the active set, at most
template <int R, bool RAVE>
__device__ __forceinline__ void active_counts(const ActiveSet<R> &s, float ep, uint32_t uvl, uint32_t T, int m,
                                              int (&out)[R], int lane) {
    const float tau = key_score(T);
#pragma unroll
    for (int r = 0; r < R; r++) {
        out[r] = 0;
        if (r >= s.rounds) continue;  // uniform
        // invariant: lo_c entries are known to be at or above T, the entry number hi_c is known
        // not to be (or hi_c is the cap)
        int lo_c = 0, hi_c = 0;
        bool up = false, galloping = false;  // the gallop away from the estimate: direction, still under way
        int step = 2;
        if (s.c[r] >= 0 && s.head[r] >= T) {
            lo_c = 1;  // the first entry itself is at or above T
            hi_c = m;
            int g = predict_count<RAVE>(s.n[r], s.w[r], s.p[r], s.vl[r], s.q2[r], ep, uvl, tau, m);
            g = g < lo_c ? lo_c : (g > hi_c ? hi_c : g);
            uint32_t kk, pp;
            if (g > lo_c) {
                entry_key<R, RAVE>(s.n[r], s.w[r], s.p[r], s.vl[r], s.q2[r], ep, uvl, g - 1, s.c[r], kk, pp);
                if (kk >= T) lo_c = g;
                else hi_c = g - 1;
            }
            if (lo_c == g && g < hi_c) {
                entry_key<R, RAVE>(s.n[r], s.w[r], s.p[r], s.vl[r], s.q2[r], ep, uvl, g, s.c[r], kk, pp);
                if (kk >= T) lo_c = g + 1;
                else hi_c = g;
            }
            if (lo_c < hi_c) {
                up = lo_c > g;
                galloping = true;
                for (; lo_c < hi_c && step <= 8; step <<= 1) {
                    int t = up ? lo_c + step : hi_c - step + 1;
                    t = t > hi_c ? hi_c : (t <= lo_c ? lo_c + 1 : t);
                    entry_key<R, RAVE>(s.n[r], s.w[r], s.p[r], s.vl[r], s.q2[r], ep, uvl, t - 1, s.c[r], kk, pp);
                    const bool ge = kk >= T;
                    if (ge) lo_c = t;
                    else hi_c = t - 1;
                    if (ge != up) {
                        galloping = false;
                        break;
                    }
                }
            }
        }
        // still far open: the whole wavefront on one child at a time
        uint64_t open = __ballot(hi_c - lo_c > kWave);
        if (__popcll(open) <= kCoopCountMax) {
            while (open != 0ull) {
                const int src = __ffsll((long long)open) - 1;
                open &= open - 1ull;
                const int cn = __builtin_amdgcn_readlane(s.n[r], src), cvl = __builtin_amdgcn_readlane(s.vl[r], src);
                const int cc = __builtin_amdgcn_readlane(s.c[r], src);
                const float cw = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s.w[r]), src));
                const float cp = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s.p[r]), src));
                const float cq2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s.q2[r]), src));
                int lo0 = __builtin_amdgcn_readlane(lo_c, src), hi0 = __builtin_amdgcn_readlane(hi_c, src);
                while (lo0 < hi0) {
                    const int step = (hi0 - lo0 + kWave - 1) / kWave;
                    const int cand = lo0 + (lane + 1) * step;  // a count: its last entry is number cand - 1
                    bool ge = false;
                    if (cand <= hi0) {
                        uint32_t kk, pp;
                        entry_key<R, RAVE>(cn, cw, cp, cvl, cq2, ep, uvl, cand - 1, cc, kk, pp);
                        ge = kk >= T;
                    }
                    const uint64_t gm = __ballot(ge);
                    const int n_ge = gm == ~0ull ? kWave : __builtin_ctzll(~gm);  // leading run of successes
                    const int new_lo = lo0 + n_ge * step;
                    const int new_hi = lo0 + (n_ge + 1) * step - 1;
                    lo0 = new_lo < hi0 ? new_lo : hi0;
                    hi0 = new_hi < hi0 ? new_hi : hi0;
                }
                if (lane == src) lo_c = hi_c = lo0;
            }
        }
        if (lo_c < hi_c) {
            // gallop on from where the three steps above left off, then bisect
            uint32_t kk, pp;
            if (galloping) {
                for (; lo_c < hi_c; step <<= 1) {
                    int t = up ? lo_c + step : hi_c - step + 1;
                    t = t > hi_c ? hi_c : (t <= lo_c ? lo_c + 1 : t);
                    entry_key<R, RAVE>(s.n[r], s.w[r], s.p[r], s.vl[r], s.q2[r], ep, uvl, t - 1, s.c[r], kk, pp);
                    const bool ge = kk >= T;
                    if (ge) lo_c = t;
                    else hi_c = t - 1;
                    if (ge != up) break;
                }
            }
            while (lo_c < hi_c) {
                int t = (lo_c + hi_c + 1) >> 1;
                entry_key<R, RAVE>(s.n[r], s.w[r], s.p[r], s.vl[r], s.q2[r], ep, uvl, t - 1, s.c[r], kk, pp);
                if (kk >= T) lo_c = t;
                else hi_c = t - 1;
            }
        }
        out[r] = lo_c;
    }
}

// The visitors of a crowded node in batches (see the file header).  On success cnt[r]
// holds the visitors of every child and sc_child / sc_occ hold (child, visit number) of
// every visitor; returns false when the node has to be replayed one visitor at a time
// (the caller's statistics are untouched either way).
//
// One batch: pick a score threshold (estimated so that about `target` unsettled entries
// lie at or above it), count EXACTLY how many entries of every child lie at or above it
// (estimate, then test the two entries around the estimate), evaluate these entries into
// LDS, sort them, and keep the first `remaining` of them when this is the last batch.
// The threshold does not have to be anything in particular: whatever it is, the entries at
// or above it are played before every entry below it, provided the checks hold.
//
// The visitors settled are those with ranks [rank0, rank0 + todo) of the node's winner
// order, starting from the state in which child i has had tk0[i] visits already (all zero
// and rank0 = 0 for a whole node; a slice of a heavy node otherwise).
template <int R, bool RAVE>
__device__ __forceinline__ bool water_level(const SelectArgs &a, const NodeCtx &c, int lane, const Kids<R, RAVE> &k,
                                            int off, int rank0, int todo, const int (&tk0)[R], WaveLds<R> &lds,
                                            int (&cnt)[R], bool allow_lds, int &lds_cur, bool use_preset,
                                            const int (&preset)[R], uint32_t *order, bool &pending) {
    lds_cur = -1;
    constexpr int F = R * kWave;
    const uint32_t uvl = (uint32_t)a.vl;
    const int m = todo;
    off += rank0;

    int tk[R];                    // visits settled so far, per child
    uint32_t headk[R], headp[R];  // the entry each child shows next
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i = r * kWave + lane;
        tk[r] = tk0[r];
        if (tk0[r] > 0 && k.part[r]) {
            entry_key<R, RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.q2[r], c.ep, uvl, tk0[r], i, headk[r], headp[r]);
        } else if (k.k2[r] > k.k1[r]) {
            headk[r] = k.k2[r];
            headp[r] = (uint32_t)(F + i);
        } else {
            headk[r] = k.k1[r];
            headp[r] = (uint32_t)i;
        }
        lds.st_n[i] = k.n[r];
        lds.st_w[i] = k.w[r];
        lds.st_p[i] = k.p[r];
        lds.st_q2[i] = k.q2[r];
    }

    // Set when the threshold search finds the unsettled entries piled up on ONE key in several
    // children and nothing above it (children exactly tied on a plateau): among equal keys the
    // lowest position wins for as long as its key stays there, so the next winners are a run of
    // the best child however short, and the next round takes it.
    bool force_run = false;
    for (int done = 0; done < m;) {
        const int remaining = m - done;
        const int run_min = force_run ? 1 : kRunShortcutMin;
        force_run = false;

        // ---- 1. threshold and exact per-child counts ----
        uint32_t lbk = 0u, lbp = 0xFFFFFFFFu;
#pragma unroll
        for (int r = 0; r < R; r++)
            if (headk[r] != 0u && comes_before(headk[r], headp[r], lbk, lbp)) {
                lbk = headk[r];
                lbp = headp[r];
            }
        uint32_t hi_key, hi_pos;
        wave_best(lbk, lbp, hi_key, hi_pos);
        if (hi_key == 0u) return false;
        const int best = (int)(hi_pos >= (uint32_t)F ? hi_pos - (uint32_t)F : hi_pos);

        // A slice of a heavy node knows exactly how many entries every child contributes to its
        // (first) batch: the entries between its two thresholds.  Nothing to search then.
        int total = 0;
        int capped_child = -1, capped_last = 0;
        bool preset_done = false;
        if (use_preset && done == 0) {
            int sum = 0;
#pragma unroll
            for (int r = 0; r < R; r++) sum += preset[r];
            total = wave_sum_i32(sum);
            if (total >= 1 && total <= kBatchCap) {
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const int i = r * kWave + lane;
                    lds.st_vl[i] = (int)((uint32_t)k.vl[r] + (uint32_t)tk[r] * uvl);
                    lds.st_j0[i] = tk[r];
                    lds.pay[i] = (uint32_t)preset[r];
                }
                wave_sync_memory();
                preset_done = true;
            }
        }
        if (!preset_done) {
        // ---- 0. a long run of the best child ----
        // When the best child's next entries stay ahead of every other child's next entry (its
        // score hardly moves with virtual loss, e.g. a RAVE blend that dominates), they are the
        // next winners one after another: count them, check them, emit them without sorting.
        if (remaining >= run_min) {
            uint32_t ok2 = 0u, opos2 = 0xFFFFFFFFu;
#pragma unroll
            for (int r = 0; r < R; r++)
                if (r * kWave + lane != best && headk[r] != 0u && comes_before(headk[r], headp[r], ok2, opos2)) {
                    ok2 = headk[r];
                    opos2 = headp[r];
                }
            uint32_t sk, spos;
            wave_best(ok2, opos2, sk, spos);
            int tn = 0, tvl = 0, ttk = 0;
            float tw = 0.0f, tp = 0.0f, tq2 = 0.0f;
#pragma unroll
            for (int r = 0; r < R; r++) {
                if (r == (best >> 6)) {
                    tn = k.n[r];
                    tw = k.w[r];
                    tp = k.p[r];
                    tvl = k.vl[r];
                    tq2 = k.q2[r];
                    ttk = tk[r];
                }
            }
            const int bl = best & 63;
            const int bn = __builtin_amdgcn_readlane(tn, bl);
            const float bw = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tw), bl));
            const float bp = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tp), bl));
            const int bvl = __builtin_amdgcn_readlane(tvl, bl);
            const float bq2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tq2), bl));
            const int btk = __builtin_amdgcn_readlane(ttk, bl);
            // probe: does the run reach kRunShortcutMin entries at all?
            uint32_t pk_, pp_;
            entry_key<R, RAVE>(bn, bw, bp, bvl, bq2, c.ep, uvl, btk + run_min - 1, best, pk_, pp_);
            if (pk_ != 0u && (sk == 0u || comes_before(pk_, pp_, sk, spos))) {
                // largest L <= remaining whose last entry still comes before the others' best
                // (64 candidate lengths at a time, one per lane; the entries are checked one by
                // one below, so this search only has to propose)
                int lo_l = run_min, hi_l = remaining;
                while (lo_l < hi_l) {
                    const int step = (hi_l - lo_l + kWave - 1) / kWave;
                    const int cand = lo_l + (lane + 1) * step;
                    bool okc = false;
                    if (cand <= hi_l) {
                        entry_key<R, RAVE>(bn, bw, bp, bvl, bq2, c.ep, uvl, btk + cand - 1, best, pk_, pp_);
                        okc = pk_ != 0u && (sk == 0u || comes_before(pk_, pp_, sk, spos));
                    }
                    const uint64_t okm = __ballot(okc);
                    const int n_ok = okm == ~0ull ? kWave : __builtin_ctzll(~okm);  // leading run of successes
                    const int new_lo = lo_l + n_ok * step;
                    const int new_hi = lo_l + (n_ok + 1) * step - 1;
                    lo_l = new_lo < hi_l ? new_lo : hi_l;
                    hi_l = new_hi < hi_l ? new_hi : hi_l;
                }
                const int L = lo_l;
                // the entry after the run must not come before the run's last one
                uint32_t nk, np2, lk_, lp_;
                entry_key<R, RAVE>(bn, bw, bp, bvl, bq2, c.ep, uvl, btk + L, best, nk, np2);
                entry_key<R, RAVE>(bn, bw, bp, bvl, bq2, c.ep, uvl, btk + L - 1, best, lk_, lp_);
                bool bad_run = nk != 0u && comes_before(nk, np2, lk_, lp_);
                // every entry of the run is checked (unless the order of the child's keys is proven
                // beforehand) and written; a long run with the helpers
                const bool proven = keys_provably_monotone<RAVE>(bn, bw, bp, bvl, bq2, c.ep, uvl, btk + L);
                if (!bad_run) {
                    if (lane == 0) lds.red[2] = 0u;
                    if (L >= 2 * kTeamMin) {
                        close_pending(pending);
                        if (lane == 0) {
                            TeamCmd &cm = lds.cmd;
                            cm.op = kOpRun;
                            cm.rounds = R;
                            cm.total = L;
                            cm.goff = off + done;
                            cm.ep = c.ep;
                            cm.uvl = uvl;
                            cm.best = best;
                            cm.btk = btk;
                            cm.bn = bn;
                            cm.bvl = bvl;
                            cm.bw = bw;
                            cm.bp = bp;
                            cm.bq2 = bq2;
                            cm.hk = hi_key;
                            cm.hp = hi_pos;
                            cm.sk = sk;
                            cm.spos = spos;
                            cm.proven = proven ? 1 : 0;
                        }
                        __syncthreads();
                        batch_run<R, RAVE, kTeam>(a, lds, lane, L, off + done, best, btk, bn, bw, bp, bvl, bq2, c.ep, uvl,
                                                  hi_key, hi_pos, sk, spos, proven);
                        __syncthreads();
                    } else {
                        wave_sync_memory();
                        batch_run<R, RAVE, kWave>(a, lds, lane, L, off + done, best, btk, bn, bw, bp, bvl, bq2, c.ep, uvl,
                                                  hi_key, hi_pos, sk, spos, proven);
                    }
                    bad_run = (lds.red[2] & 4u) != 0u;
                }
                if (!bad_run) {
                    if (lane == bl) {
#pragma unroll
                        for (int r = 0; r < R; r++)
                            if (r == (best >> 6)) {
                                tk[r] = btk + L;
                                headk[r] = nk;
                                headp[r] = np2;
                            }
                    }
                    done += L;
                    continue;
                }
            }
        }
        if (run_min == 1) return false;  // the run that had to be there was refused
        const int want = remaining < kBatchCap ? remaining : kBatchCap;
        // lower bound of any useful threshold: a child alone has `want` entries at or above the
        // key of its want-th next visit; the best such key over all children (the child that
        // holds out longest, which need not be the one with the best next entry)
        uint32_t lo_key = 0u;
        {
            uint32_t lmax = 0u;
#pragma unroll
            for (int r = 0; r < R; r++) {
                if (k.part[r] && headk[r] != 0u) {
                    uint32_t kk, pp;
                    entry_key<R, RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.q2[r], c.ep, uvl, tk[r] + want - 1,
                                       r * kWave + lane, kk, pp);
                    lmax = umax32(lmax, kk);
                }
            }
            lo_key = wave_max_u32(lmax);
        }
        if (lo_key == 0u) lo_key = 1u;
        if (lo_key > hi_key) return false;  // scores rose along the best child's list

        // Only children whose next entry reaches the lower bound can contribute.  They are
        // listed densely (one per lane and round), so that the work below costs one round per
        // 64 ACTIVE children instead of one per 64 children.
        int n_act = 0;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int i = r * kWave + lane;
            const bool act = headk[r] != 0u && headk[r] >= lo_key;
            const uint64_t am = __ballot(act);
            if (act) lds.pay2[1][n_act + __popcll(am & ((1ull << lane) - 1ull))] = (uint32_t)i;
            n_act += __popcll(am);
            lds.key[1][i] = headk[r];  // key of the child's next entry
            lds.st_vl[i] = (int)((uint32_t)k.vl[r] + (uint32_t)tk[r] * uvl);
            lds.st_j0[i] = tk[r];
            lds.pay[i] = 0u;  // result: entries of the batch
        }
        wave_sync_memory();
        const int rounds = (n_act + kWave - 1) / kWave;
        int an[R], avl[R], ac[R];
        float aw[R], ap[R], aq2[R];
        uint32_t ahead[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            ac[r] = -1;
            an[r] = 0;
            avl[r] = 0;
            aw[r] = ap[r] = aq2[r] = 0.0f;
            ahead[r] = 0u;
            if (r < rounds && r * kWave + lane < n_act) {
                const int ci = (int)lds.pay2[1][r * kWave + lane];
                ac[r] = ci;
                an[r] = lds.st_n[ci];
                aw[r] = lds.st_w[ci];
                ap[r] = lds.st_p[ci];
                avl[r] = lds.st_vl[ci];
                aq2[r] = lds.st_q2[ci];
                ahead[r] = lds.key[1][ci];
            }
        }
        // the estimate is off by about one entry per active child: aim a margin above what is
        // needed when this can be the last batch, a margin below the capacity otherwise
        const int margin = n_act + 8;
        const bool can_finish = remaining + 2 * margin <= kBatchCap;
        int target = can_finish ? remaining + margin : kBatchCap - margin;
        if (target < 1) return false;
        // No child can win more than the visits that are left: its entries beyond that are
        // never looked at (the batch is cut at `remaining` entries anyway, and such a child's
        // last counted entry lies at or after that cut).
        const int child_cap = remaining < kBatchCap + 1 ? remaining : kBatchCap + 1;
        int ct[R];
        total = 0;
        int tries = 0;
        uint32_t T_forced = 0u;  // threshold imposed for the next round instead of searching one
        bool allow_above = true;
        for (;;) {
            if (++tries > 8) return false;
            const uint32_t T_now = T_forced;  // imposed for this round only
            T_forced = 0u;
            // a threshold with about `target` ESTIMATED entries at or above it (no exact evaluation
            // yet): a quarter more than aimed at costs less than more search steps, and a batch that
            // cannot finish the node anyway may as well be a little smaller
            uint32_t klo = lo_key;
            int n_evals = 0;
            if (T_now == 0u) {
                int acc_hi = target + (target >> 2);
                if (acc_hi > kBatchCap - margin) acc_hi = kBatchCap - margin;
                if (acc_hi < target) acc_hi = target;
                const int acc_below = can_finish ? target : target - (target >> 2);
                klo = search_threshold(lo_key, hi_key, target, acc_hi, acc_below, n_evals, [&](uint32_t kmid) {
                    const float mid = key_score(kmid);
                    int est = 0;
#pragma unroll
                    for (int r = 0; r < R; r++)
                        if (r < rounds && ac[r] >= 0)
                            est += predict_count<RAVE>(an[r], aw[r], ap[r], avl[r], aq2[r], c.ep, uvl, mid, child_cap);
                    return wave_sum_i32(est);
                });
            }
            uint32_t T = T_now != 0u ? T_now : klo;
            if (T < lo_key) T = lo_key;
            if (T > hi_key) T = hi_key;
            const float tau = key_score(T);
            // exact count of every active child at T: test the two entries around the estimate
            int sum = 0;
#pragma unroll
            for (int r = 0; r < R; r++) {
                ct[r] = 0;
                if (r < rounds && ac[r] >= 0 && ahead[r] >= T) {
                    int lo_c = 1, hi_c = child_cap;  // the next entry itself is at or above T
                    int g = predict_count<RAVE>(an[r], aw[r], ap[r], avl[r], aq2[r], c.ep, uvl, tau, child_cap);
                    g = g < lo_c ? lo_c : (g > hi_c ? hi_c : g);
                    uint32_t kk, pp;
                    if (g > lo_c) {
                        entry_key<R, RAVE>(an[r], aw[r], ap[r], avl[r], aq2[r], c.ep, uvl, g - 1, ac[r], kk, pp);
                        if (kk >= T) lo_c = g;
                        else hi_c = g - 1;
                    }
                    if (lo_c == g && g < hi_c) {
                        entry_key<R, RAVE>(an[r], aw[r], ap[r], avl[r], aq2[r], c.ep, uvl, g, ac[r], kk, pp);
                        if (kk >= T) lo_c = g + 1;
                        else hi_c = g;
                    }
                    // estimate off by more than one: gallop away from it, then bisect what is left
                    if (lo_c < hi_c) {
                        const bool up = lo_c > g;
                        for (int step = 2; lo_c < hi_c; step <<= 1) {
                            int t = up ? lo_c + step : hi_c - step + 1;
                            t = t > hi_c ? hi_c : (t <= lo_c ? lo_c + 1 : t);
                            entry_key<R, RAVE>(an[r], aw[r], ap[r], avl[r], aq2[r], c.ep, uvl, t - 1, ac[r], kk, pp);
                            const bool ge = kk >= T;
                            if (ge) lo_c = t;
                            else hi_c = t - 1;
                            if (ge != up) break;
                        }
                    }
                    while (lo_c < hi_c) {
                        int t = (lo_c + hi_c + 1) >> 1;
                        entry_key<R, RAVE>(an[r], aw[r], ap[r], avl[r], aq2[r], c.ep, uvl, t - 1, ac[r], kk, pp);
                        if (kk >= T) lo_c = t;
                        else hi_c = t - 1;
                    }
                    ct[r] = lo_c;
                    sum += lo_c;
                }
            }
            total = wave_sum_i32(sum);  // at most 64 * R * (capacity + 1)
            if (a.stats && lane == 0) atomicAdd(a.stats + 5, 1);
            // A batch that does not fit is cut at the child with most entries (typically one
            // whose score hardly moves with virtual loss): it contributes fewer entries now,
            // and the batch is later cut right after its last one.
            capped_child = -1;
            capped_last = 0;
            if (total > kBatchCap) {
                int mx = 0, mi = -1;
#pragma unroll
                for (int r = 0; r < R; r++)
                    if (ct[r] > mx) {
                        mx = ct[r];
                        mi = ac[r];
                    }
                const uint32_t gmx = wave_max_u32((uint32_t)mx);
                const int who = (int)wave_min_u32((uint32_t)mx == gmx ? (uint32_t)mi : 0xFFFFFFFFu);
                const int excess = total - kBatchCap;
                // One child floods the batch with entries AT the threshold (a score that hardly
                // moves with virtual loss).  Take the entries strictly above it first, a small
                // batch; the run of that child is then emitted without sorting.
                if (allow_above && T < hi_key && ((int)gmx > excess || tries >= 3)) {
                    // (after a few rounds of aiming higher in vain the key is taken to be flooded by
                    // several children at once)
                    allow_above = false;
                    T_forced = T + 1u;
                    continue;
                }
                if (T >= hi_key) {
                    force_run = true;  // flooded at the best key itself: nothing lies above, the best child runs
                    break;
                }
                if ((int)gmx <= excess) {
                    target -= excess + margin;  // no single child absorbs it: aim higher instead
                    if (target < 1) target = 1;
                    continue;
                }
#pragma unroll
                for (int r = 0; r < R; r++)
                    if (ac[r] == who) ct[r] -= excess;
                capped_child = who;
                total = kBatchCap;
            }
            if (T_now != 0u) {
                // nothing above the flooded key: every child's next entry is at that key or below,
                // equal keys go by position, so the best child runs first, however short its run
                // (the child that floods the key follows with a long one)
                if (total < 1) force_run = true;
                break;  // may not finish the node: the run comes next
            }
            if (can_finish && total < remaining) {
                target += (remaining - total) + margin;  // not enough to finish: aim lower
                if (target > kBatchCap) return false;
                continue;
            }
            if (total < 1) return false;
            break;
        }
        if (force_run) continue;
        // hand the counts back to the lanes that own the children
#pragma unroll
        for (int r = 0; r < R; r++)
            if (ac[r] >= 0) lds.pay[ac[r]] = (uint32_t)ct[r];
        wave_sync_memory();
        }  // !preset_done
        int nb[R];  // entries of every own child in this batch
#pragma unroll
        for (int r = 0; r < R; r++) nb[r] = (int)lds.pay[r * kWave + lane];
        if (capped_child >= 0) capped_last = lds.st_j0[capped_child] + (int)lds.pay[capped_child] - 1;
        wave_sync_memory();

        // ---- 2. evaluate the batch in (child, visit) order ----
        int carry = 0;
#pragma unroll
        for (int r = 0; r < R; r++) {
            int inc = wave_inclusive_sum(nb[r], lane);
            lds.offs[r * kWave + lane] = carry + inc - nb[r];
            carry += __builtin_amdgcn_readlane(inc, 63);
        }
        wave_sync_memory();
        // ---- 2./3. evaluate the batch and put it in winner order; a batch that is worth it
        // is shared with the helper wavefronts of the block ----
        const bool team = total >= kTeamMin;
        int cur;
        if (team) {
            close_pending(pending);
            if (lane == 0) {
                lds.cmd.op = kOpOrder;
                lds.cmd.rounds = R;
                lds.cmd.total = total;
                lds.cmd.ep = c.ep;
                lds.cmd.uvl = uvl;
            }
            __syncthreads();
            cur = batch_order<R, RAVE, kTeam>(lds, lane, total, c.ep, uvl);
            __syncthreads();
        } else {
            cur = batch_order<R, RAVE, kWave>(lds, lane, total, c.ep, uvl);
        }
        if ((lds.red[2] & 4u) != 0u) return false;
        const uint32_t *skey = lds.key[cur], *spay = lds.pay2[cur];

        // ---- 4. winner order: keep what is needed, check ties across children, emit ----
        int keep = total < remaining ? total : remaining;
        if (capped_child >= 0) {
            // position of the capped child's last evaluated entry in the sorted batch
            uint32_t qcut = 0xFFFFFFFFu;
            const uint32_t want_pay = ((uint32_t)capped_child << 21) | (uint32_t)capped_last;
            for (int q = lane; q < total; q += kWave) {
                if ((spay[q] & 0x7FFFFFFFu) == want_pay) qcut = umin32(qcut, (uint32_t)q);
            }
            qcut = wave_min_u32(qcut);
            if (qcut == 0xFFFFFFFFu) return false;
            if ((int)qcut + 1 < keep) keep = (int)qcut + 1;
        }
        // a node that this one batch settles keeps its winner order in LDS for the partition
        const bool only_batch = allow_lds && done == 0 && keep == m;
        if (team) {
            close_pending(pending);
            if (lane == 0) {
                lds.cmd.op = kOpEmit;
                lds.cmd.rounds = R;
                lds.cmd.total = total;
                lds.cmd.keep = keep;
                lds.cmd.goff = only_batch ? -1 : off + done;
                lds.cmd.cur = cur;
            }
            __syncthreads();
            batch_emit<R, kTeam>(a, lds, order, lane, total, keep, only_batch ? -1 : off + done, cur);
            __syncthreads();
        } else {
            if (only_batch) close_pending(pending);  // the previous node's partition may still read the order
            batch_emit<R, kWave>(a, lds, order, lane, total, keep, only_batch ? -1 : off + done, cur);
        }
        if (only_batch) lds_cur = 0;
        bool bad = (lds.red[2] & 4u) != 0u;
        wave_sync_memory();
        {
            // The last kept entry must come before every child's first unevaluated entry (a
            // child with dropped entries is covered by the order check above), and that entry
            // must not come before the child's own last evaluated one.
            const uint32_t lk = ~skey[keep - 1];
            const uint32_t lpay = spay[keep - 1];
            const uint32_t lchild = (lpay >> 21) & 1023u;
            const uint32_t lpos = lchild + ((lpay >> 31) ? (uint32_t)F : 0u);
#pragma unroll
            for (int r = 0; r < R; r++) {
                const int i = r * kWave + lane;
                const int settled = lds.hist[i] > tk[r] ? lds.hist[i] : tk[r];
                uint32_t uk = headk[r], up = headp[r];
                if (k.part[r] && nb[r] > 0) {
                    entry_key<R, RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.q2[r], c.ep, uvl, tk[r] + nb[r], i, uk, up);
                    uint32_t ek, ep2;
                    entry_key<R, RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.q2[r], c.ep, uvl, tk[r] + nb[r] - 1, i, ek,
                                       ep2);
                    if (ek == 0u || comes_before(uk, up, ek, ep2)) bad = true;
                }
                if (k.part[r] && uk != 0u && (uint32_t)i != lchild && !comes_before(lk, lpos, uk, up)) bad = true;
                // the child's next entry after this batch
                if (k.part[r] && settled > tk[r]) {
                    if (settled == tk[r] + nb[r]) {
                        headk[r] = uk;
                        headp[r] = up;
                    } else {
                        entry_key<R, RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.q2[r], c.ep, uvl, settled, i, headk[r],
                                           headp[r]);
                    }
                }
                tk[r] = settled;
            }
        }
        if (__ballot(bad) != 0ull) return false;
        done += keep;
        wave_sync_memory();
    }
#pragma unroll
    for (int r = 0; r < R; r++) cnt[r] = tk[r];
    return true;
}

// A threshold at or above which about `target` of the node's entries lie, found on ESTIMATED
// counts (search_threshold).  The thresholds of a node's targets come out ordered like the
// targets: a search either stops with its count inside [target, target + window], and the windows
// of two targets are narrower than their distance, or it ends on the largest key whose count
// still reaches the target; the counts do not increase with the key, so in every combination the
// larger target gets the lower key.  (The estimate's fast arithmetic may break that monotonicity
// by a hair; the caller checks the order of the thresholds and of the exact counts.)
//
// A target whose rank falls inside the run of ONE child whose key hardly moves with virtual loss (a RAVE
// blend that dominates: thousands of its entries within a few hundred keys, or on one key) cannot be met by
// looking at estimated counts: they jump from far below to far above the target between neighbouring
// keys, and the estimate for that child is the ill-conditioned one.  When six steps have not met the
// window and one child accounts for most of the difference between the counts at the two ends of the
// bracket, the threshold is taken from that child's own list instead: the EXACT key of its entry number
// target - (what the others have at the upper end), which puts about `target` entries at or above it
// whatever the estimate said about the child itself.  Still a function of the node and the target only,
// and decreasing in the target (the child's keys do not increase), so neighbouring slices agree and the
// order of the thresholds holds; the callers check both anyway.
template <int R, bool RAVE>
__device__ __forceinline__ uint32_t active_threshold(const ActiveSet<R> &s, float ep, uint32_t uvl, uint32_t lo_key,
                                                     uint32_t hi_key, int target, int window, int m, int lane) {
    int n_evals = 0;
    return search_threshold(
        lo_key, hi_key, target, target + window, target, n_evals,
        [&](uint32_t kmid) {
            const float mid = key_score(kmid);
            int est = 0;
#pragma unroll
            for (int r = 0; r < R; r++)
                if (r < s.rounds && s.c[r] >= 0)
                    est += predict_count<RAVE>(s.n[r], s.w[r], s.p[r], s.vl[r], s.q2[r], ep, uvl, mid, m);
            return wave_sum_i32(est);
        },
        [&](uint32_t klo, uint32_t khi) {
            const float tlo = key_score(klo), thi = key_score(khi);
            // the child whose estimated count differs most between the two ends (lowest child on ties)
            uint32_t best = 0u;  // (difference << 10) | (1023 - slot in the active set): the largest wins
            int my_hi[R];
            int sum_lo = 0, sum_hi = 0;
#pragma unroll
            for (int r = 0; r < R; r++) {
                my_hi[r] = 0;
                if (r < s.rounds && s.c[r] >= 0) {
                    const int a = predict_count<RAVE>(s.n[r], s.w[r], s.p[r], s.vl[r], s.q2[r], ep, uvl, tlo, m);
                    my_hi[r] = predict_count<RAVE>(s.n[r], s.w[r], s.p[r], s.vl[r], s.q2[r], ep, uvl, thi, m);
                    sum_lo += a;
                    sum_hi += my_hi[r];
                    const int d = a - my_hi[r] > 0 ? a - my_hi[r] : 0;
                    const uint32_t v = ((uint32_t)(d > 0x1FFFFF ? 0x1FFFFF : d) << 10) | (uint32_t)(1023 - (r * kWave + lane));
                    best = best > v ? best : v;
                }
            }
            const int e_lo = wave_sum_i32(sum_lo), e_hi = wave_sum_i32(sum_hi);
            const uint32_t top = wave_max_u32(best);
            const int d_top = (int)(top >> 10), slot = 1023 - (int)(top & 1023u);
            // no single child behind the jump, or the target is not between the ends
            if (top == 0u || e_lo < target || e_hi >= target || (long long)d_top * 10 < (long long)(e_lo - e_hi) * 6) return 0u;
            const int src = slot & 63;
            int an = 0, avl = 0, ac = 0, ah = 0;
            float aw = 0.0f, ap = 0.0f, aq2 = 0.0f;
#pragma unroll
            for (int r = 0; r < R; r++)
                if (r == (slot >> 6)) {
                    an = s.n[r];
                    avl = s.vl[r];
                    ac = s.c[r];
                    ah = my_hi[r];
                    aw = s.w[r];
                    ap = s.p[r];
                    aq2 = s.q2[r];
                }
            an = __builtin_amdgcn_readlane(an, src);
            avl = __builtin_amdgcn_readlane(avl, src);
            ac = __builtin_amdgcn_readlane(ac, src);
            ah = __builtin_amdgcn_readlane(ah, src);
            aw = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(aw), src));
            ap = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ap), src));
            aq2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(aq2), src));
            const int ja = target - (e_hi - ah);  // entries of that child wanted at or above the threshold
            if (ac < 0 || ja < 1 || ja > m) return 0u;
            uint32_t kk, pp;
            entry_key<R, RAVE>(an, aw, ap, avl, aq2, ep, uvl, ja - 1, ac, kk, pp);
            return kk;
        });
}

// For a slice of a heavy node: the boundary of the cumulative target `target`: a threshold key T
// and EXACTLY how many entries of every own child lie above the boundary (ct; at most m each, m >= target:
// a cap on what is looked at, not the node's visitor count, of which a boundary does not depend): the
// entries at or above T, or, where far more entries than the target pile up on T itself, those over T and
// the first of the pile (see below).  Deterministic, a function of the node's state and the target only.
// Uses the LDS scratch.
template <int R, bool RAVE>
__device__ __forceinline__ bool threshold_counts(const SelectArgs &a, const NodeCtx &c, int lane,
                                                 const Kids<R, RAVE> &k, WaveLds<R> &lds, int m, int window,
                                                 int target, int (&ct)[R], uint32_t &T) {
    constexpr int F = R * kWave;
    const uint32_t uvl = (uint32_t)a.vl;
    uint32_t headk[R];
    uint32_t lbk = 0u, lbp = 0xFFFFFFFFu;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i = r * kWave + lane;
        uint32_t hp;
        if (k.k2[r] > k.k1[r]) {
            headk[r] = k.k2[r];
            hp = (uint32_t)(F + i);
        } else {
            headk[r] = k.k1[r];
            hp = (uint32_t)i;
        }
        if (headk[r] != 0u && comes_before(headk[r], hp, lbk, lbp)) {
            lbk = headk[r];
            lbp = hp;
        }
    }
    uint32_t hi_key, hi_pos;
    wave_best(lbk, lbp, hi_key, hi_pos);
    if (hi_key == 0u) return false;
    // A child alone has m entries at or above the key of its m-th visit: the best such key over
    // all children is a lower bound for every threshold of the node.
    uint32_t lo_key = 0u;
    {
        uint32_t lmax = 0u;
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (k.part[r] && headk[r] != 0u) {
                uint32_t kk, pp;
                entry_key<R, RAVE>(k.n[r], k.w[r], k.p[r], k.vl[r], k.q2[r], c.ep, uvl, m - 1, r * kWave + lane, kk, pp);
                lmax = umax32(lmax, kk);
            }
        }
        lo_key = wave_max_u32(lmax);
    }
    if (lo_key == 0u) lo_key = 1u;
    if (lo_key > hi_key) return false;
    // the active children, densely
    int n_act = 0;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i = r * kWave + lane;
        const bool act = k.part[r] && headk[r] != 0u && headk[r] >= lo_key;
        const uint64_t am = __ballot(act);
        if (act) lds.pay2[1][n_act + __popcll(am & ((1ull << lane) - 1ull))] = (uint32_t)i;
        n_act += __popcll(am);
        lds.key[1][i] = headk[r];
        lds.st_n[i] = k.n[r];
        lds.st_w[i] = k.w[r];
        lds.st_p[i] = k.p[r];
        lds.st_vl[i] = k.vl[r];
        lds.st_q2[i] = k.q2[r];
        lds.pay[i] = 0u;
    }
    wave_sync_memory();
    ActiveSet<R> s;
    s.rounds = (n_act + kWave - 1) / kWave;
#pragma unroll
    for (int r = 0; r < R; r++) {
        s.c[r] = -1;
        s.n[r] = 0;
        s.vl[r] = 0;
        s.w[r] = s.p[r] = s.q2[r] = 0.0f;
        s.head[r] = 0u;
        if (r < s.rounds && r * kWave + lane < n_act) {
            const int ci = (int)lds.pay2[1][r * kWave + lane];
            s.c[r] = ci;
            s.n[r] = lds.st_n[ci];
            s.w[r] = lds.st_w[ci];
            s.p[r] = lds.st_p[ci];
            s.vl[r] = lds.st_vl[ci];
            s.q2[r] = lds.st_q2[ci];
            s.head[r] = lds.key[1][ci];
        }
    }
    int cta[R];
    {
    // The boundary of one target: the threshold and the exact counts at it.  When far more entries than the
    // target lie at or above the threshold, they are piled up ON the threshold key (a child whose key does not
    // move at all over hundreds of visits; no key separates them), and the boundary is put inside the pile:
    // entries of one key are played child after child by position (first-scan candidates in child order, then
    // second-scan candidates; comes_before), each child's in visit order, so the first `target - above` of the
    // pile in that order belong above the boundary, where `above` counts the entries at keys over the threshold
    // (none of the pile when `above` reaches the target by itself).  The counts that come out add up to
    // max(target, above); they are still a function of the node and the target alone, and grow with the target:
    // two targets with one threshold share `above`, and of two thresholds the lower one's `above` holds
    // everything at or above the higher one.  Whoever uses the counts checks the order they imply like any
    // other (water_level: the last entry kept must come before every child's next one).
        T = active_threshold<R, RAVE>(s, c.ep, uvl, lo_key, hi_key, target, window, m, lane);
        active_counts<R, RAVE>(s, c.ep, uvl, T, m, cta, lane);
        int sum = 0;
#pragma unroll
        for (int r = 0; r < R; r++) sum += cta[r];
        const int at_or_above = wave_sum_i32(sum);
        if (at_or_above - target > window && T < hi_key) {
            int ctb[R];  // entries at keys over the threshold
            active_counts<R, RAVE>(s, c.ep, uvl, T + 1u, m, ctb, lane);
            sum = 0;
#pragma unroll
            for (int r = 0; r < R; r++) sum += ctb[r];
            const int above = wave_sum_i32(sum);
            if (above >= target) {
                // the key above the threshold has enough already (the search works on estimates): the boundary
                // goes between the two keys
#pragma unroll
                for (int r = 0; r < R; r++) cta[r] = ctb[r];
            } else {
                // the pile: e entries of every child at the threshold key, from its visit number ctb on; where
                // the child stands in the order of the pile
                int e1[R], e2[R];
                bool odd = false;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    e1[r] = e2[r] = 0;
                    const int e = cta[r] - ctb[r];
                    if (r < s.rounds && s.c[r] >= 0 && e > 0) {
                        uint32_t kk, pp;
                        entry_key<R, RAVE>(s.n[r], s.w[r], s.p[r], s.vl[r], s.q2[r], c.ep, uvl, ctb[r], s.c[r], kk, pp);
                        if (kk != T) odd = true;
                        if (pp >= (uint32_t)F) e2[r] = e;
                        else e1[r] = e;
                    } else if (e < 0) {
                        odd = true;
                    }
                }
                if (__ballot(odd) == 0ull) {
                    int need = target - above;
                    // the active children are listed in child order: first-scan candidates first, in that order
                    int carry = 0;
                    int take[R];
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const int inc = wave_inclusive_sum(e1[r], lane);
                        const int before = carry + inc - e1[r];
                        const int left = need - before;
                        take[r] = e1[r] > 0 ? (left <= 0 ? 0 : (left < e1[r] ? left : e1[r])) : 0;
                        carry += __builtin_amdgcn_readlane(inc, 63);
                    }
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const int inc = wave_inclusive_sum(e2[r], lane);
                        const int before = carry + inc - e2[r];
                        const int left = need - before;
                        if (e2[r] > 0) take[r] = left <= 0 ? 0 : (left < e2[r] ? left : e2[r]);
                        carry += __builtin_amdgcn_readlane(inc, 63);
                    }
#pragma unroll
                    for (int r = 0; r < R; r++) cta[r] = ctb[r] + take[r];
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++)
            if (s.c[r] >= 0) lds.pay[s.c[r]] = (uint32_t)cta[r];
        wave_sync_memory();
#pragma unroll
        for (int r = 0; r < R; r++) ct[r] = (int)lds.pay[r * kWave + lane];
        wave_sync_memory();
    }
    if (a.stats && lane == 0) atomicAdd(a.stats + 5, 1);
    return true;
}

// Boundary number b of a heavy node cut into slices of S visitors (the one between slices b - 1 and b: target
// rank b * S, window S / 4), through the node's boundary table: whoever asks first works it out and leaves it
// there (ready word 2 * call number + 1; 2 * call number while it is being worked out), everybody else takes it
// from there.  One value per boundary whoever computes it: the slices on both sides, and the wavefronts that
// work boundaries out ahead of time (items of kind 4, published while the node's parent is still being settled:
// a boundary depends on the node's statistics and its rank only, not on how many visitors the node ends up
// with).  Whoever holds a claim is running and waits for nothing before it writes, so the bounded wait ends.
// Returns false when the threshold search failed, or when the selection is being given up.
template <int R, bool RAVE>
__device__ __forceinline__ bool slice_boundary(const SelectArgs &a, const NodeCtx &c, int lane, const Kids<R, RAVE> &k,
                                               WaveLds<R> &lds, int hid, int b, int S, int (&ct)[R], uint32_t &T,
                                               int &rank) {
    int *bnd = a.hbound + ((size_t)hid * kMaxSlices + (size_t)(b - 1)) * kBoundInts;  // b = 1 .. kMaxSlices
    const int claimed = 2 * a.epoch, ready = claimed + 1;
    int state = 0;  // 1 this wavefront works it out, 2 it is there
    for (int spins = 0;; spins++) {
        int got = 0, ab = 0;
        if (lane == 0) {
            const int v = __hip_atomic_load(bnd + 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (v == ready) got = 2;
            else if (v != claimed) got = atomicCAS(bnd + 0, v, claimed) == v ? 1 : 0;
            else if ((spins & 3) == 3)
                ab = __hip_atomic_load(a.sched_wait + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        got = __builtin_amdgcn_readfirstlane(got);
        ab = __builtin_amdgcn_readfirstlane(ab);
        if (got) {
            state = got;
            break;
        }
        if (ab) break;
        if (spins >= a.spin_limit) {
            if (lane == 0) atomicCAS(a.sched_wait + 1, 0, 3);
            break;
        }
        __builtin_amdgcn_s_sleep(4);
    }
    if (state == 0) return false;
    if (state == 1) {
        const bool ok = threshold_counts<R, RAVE>(a, c, lane, k, lds, b * S + S, S >> 2, b * S, ct, T);
        int sum = 0;
#pragma unroll
        for (int r = 0; r < R; r++) {
            bnd[16 + r * kWave + lane] = ct[r];
            sum += ct[r];
        }
        rank = wave_sum_i32(sum);
        if (lane == 0) {
            bnd[1] = (int)T;
            bnd[2] = rank;
            bnd[3] = ok ? 1 : 0;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        if (lane == 0) __hip_atomic_store(bnd + 0, ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return ok;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    T = (uint32_t)__hip_atomic_load(bnd + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    rank = __hip_atomic_load(bnd + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool ok = __hip_atomic_load(bnd + 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
#pragma unroll
    for (int r = 0; r < R; r++)
        ct[r] = __hip_atomic_load(bnd + 16 + r * kWave + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return ok;
}

// A boundary that another wavefront works out, taken from the table once it is there: the counts of every own
// child and their sum.  Gives up (false) after `polls` polls: only for work that can be left undone.
template <int R>
__device__ __forceinline__ bool boundary_read(const SelectArgs &a, int lane, int hid, int b, int polls, int (&ct)[R],
                                              int &rank) {
    const int *bnd = a.hbound + ((size_t)hid * kMaxSlices + (size_t)(b - 1)) * kBoundInts;
    const int ready = 2 * a.epoch + 1;
    bool there = false;
    for (int spins = 0; spins < polls; spins++) {
        int v = 0;
        if (lane == 0) v = __hip_atomic_load(bnd + 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        v = __builtin_amdgcn_readfirstlane(v);
        if (v == ready) {
            there = true;
            break;
        }
        __builtin_amdgcn_s_sleep(8);
    }
    if (!there) return false;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    rank = __hip_atomic_load(bnd + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool ok = __hip_atomic_load(bnd + 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
#pragma unroll
    for (int r = 0; r < R; r++)
        ct[r] = __hip_atomic_load(bnd + 16 + r * kWave + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return ok;
}

// The commonest crowded node: one child wins every time.  That is the case exactly when
// the score it shows to the last visitor still comes before the first score of every
// other child and its own scores never increase on the way; both are checked on the exact
// values (m evaluations spread over the lanes).  Returns false when it is not that case.
// True when entries 0 .. m-1 of a child never come before their predecessor (m evaluations
// spread over the lanes), or when the arithmetic proves it beforehand.
template <int R, bool RAVE>
__device__ __forceinline__ bool entries_in_order(int bn, float bw, float bp, int bvl, float bq2, float ep, uint32_t uvl,
                                                 int best, int m, int lane) {
    if (keys_provably_monotone<RAVE>(bn, bw, bp, bvl, bq2, ep, uvl, m - 1)) return true;
    bool bad = false;
    uint32_t carry_k = 0xFFFFFFFFu, carry_p = 0u;  // entry before the chunk
    for (int base = 0; base < m; base += kWave) {
        const int j = base + lane;
        uint32_t kk = 0u, pp = 0xFFFFFFFFu;
        if (j < m) entry_key<R, RAVE>(bn, bw, bp, bvl, bq2, ep, uvl, j, best, kk, pp);
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
    return __ballot(bad) == 0ull;
}

template <int R, bool RAVE>
__device__ __forceinline__ bool single_run(const SelectArgs &a, const NodeCtx &c, int lane, const Kids<R, RAVE> &k,
                                           uint32_t bk, uint32_t bpos, int off, int m, bool to_global, int (&cnt)[R],
                                           int &run_child, bool &contested, int &best0, uint32_t &lk0, uint32_t &lp0) {
    // contested: the best child's entry for the last visitor, (lk0, lp0), is real but does not come first
    contested = false;
    constexpr int F = R * kWave;
    const uint32_t uvl = (uint32_t)a.vl;
    uint32_t hi_key, hi_pos;
    wave_best(bk, bpos, hi_key, hi_pos);
    if (hi_key == 0u) return false;
    const int best = (int)(hi_pos >= (uint32_t)F ? hi_pos - (uint32_t)F : hi_pos);
    // statistics of the best child, wave-uniform
    int tn = 0, tvl = 0;
    float tw = 0.0f, tp = 0.0f, tq2 = 0.0f;
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (r == (best >> 6)) {
            tn = k.n[r];
            tw = k.w[r];
            tp = k.p[r];
            tvl = k.vl[r];
            tq2 = k.q2[r];
        }
    }
    const int bl = best & 63;
    const int bn = __builtin_amdgcn_readlane(tn, bl);
    const float bw = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tw), bl));
    const float bp = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tp), bl));
    const int bvl = __builtin_amdgcn_readlane(tvl, bl);
    const float bq2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tq2), bl));
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
    entry_key<R, RAVE>(bn, bw, bp, bvl, bq2, c.ep, uvl, m - 1, best, lk, lp);
    if (lk == 0u) return false;
    if (sk != 0u && !comes_before(lk, lp, sk, spos)) {
        contested = true;  // other children get a look in: the caller may still find that they are few
        best0 = best;
        lk0 = lk;
        lp0 = lp;
        return false;
    }
    // when the order of the child's keys is proven beforehand, the entries in between need no look
    if (!entries_in_order<R, RAVE>(bn, bw, bp, bvl, bq2, c.ep, uvl, best, m, lane)) return false;
    if (to_global) {
        for (int j = lane; j < m; j += kWave) {
            a.sc_child[off + j] = best;
            a.sc_occ[off + j] = j;
        }
    }
    if (lane == bl) {
#pragma unroll
        for (int r = 0; r < R; r++)
            if (r == (best >> 6)) cnt[r] = m;
    }
    run_child = best;
    return true;
}

// How many of a child's entries 0 .. cap-1 come before the entry (tk, tp), given that the child's
// keys do not increase (the caller checks the entries it then uses): the closed-form estimate,
// the two entries around it tested with the exact arithmetic, and a gallop away from it plus a
// bisection when it is further off.  first_known: entry 0 is known to come before (tk, tp).  On
// return c: entry c-1 was seen to come before (tk, tp) (or c == 0, or c == 1 with first_known),
// entry c was seen not to (or c == cap).
template <int R, bool RAVE>
__device__ __forceinline__ int count_before(int n, float w, float p, int vl, float q2, float ep, uint32_t uvl,
                                            int child, uint32_t tk, uint32_t tp, int cap, bool first_known) {
    uint32_t kk, pp;
    if (!first_known) {
        entry_key<R, RAVE>(n, w, p, vl, q2, ep, uvl, 0, child, kk, pp);
        if (!(kk != 0u && comes_before(kk, pp, tk, tp))) return 0;
    }
    int lo_c = 1, hi_c = cap;
    if (hi_c < lo_c) return lo_c;
    int g = predict_count<RAVE>(n, w, p, vl, q2, ep, uvl, key_score(tk), cap);
    g = g < lo_c ? lo_c : (g > hi_c ? hi_c : g);
    if (g > lo_c) {
        entry_key<R, RAVE>(n, w, p, vl, q2, ep, uvl, g - 1, child, kk, pp);
        if (kk != 0u && comes_before(kk, pp, tk, tp)) lo_c = g;
        else hi_c = g - 1;
    }
    if (lo_c == g && g < hi_c) {
        entry_key<R, RAVE>(n, w, p, vl, q2, ep, uvl, g, child, kk, pp);
        if (kk != 0u && comes_before(kk, pp, tk, tp)) lo_c = g + 1;
        else hi_c = g;
    }
    if (lo_c < hi_c) {
        const bool up = lo_c > g;
        for (int step = 2; lo_c < hi_c; step <<= 1) {
            int t = up ? lo_c + step : hi_c - step + 1;
            t = t > hi_c ? hi_c : (t <= lo_c ? lo_c + 1 : t);
            entry_key<R, RAVE>(n, w, p, vl, q2, ep, uvl, t - 1, child, kk, pp);
            const bool before = kk != 0u && comes_before(kk, pp, tk, tp);
            if (before) lo_c = t;
            else hi_c = t - 1;
            if (before != up) break;
        }
    }
    while (lo_c < hi_c) {
        const int t = (lo_c + hi_c + 1) >> 1;
        entry_key<R, RAVE>(n, w, p, vl, q2, ep, uvl, t - 1, child, kk, pp);
        if (kk != 0u && comes_before(kk, pp, tk, tp)) lo_c = t;
        else hi_c = t - 1;
    }
    return lo_c;
}

constexpr int kSparseMax = 64;  // entries of other children a nearly-one-winner node may hold (one per lane)
constexpr int kSparseMin = 8;    // visitors from which that direct merge is tried
static_assert(2 * kHeavyMin <= kBatchCap, "the (key, position) list of the dominant child fits one sort buffer");


// A node where one child wins ALMOST every time: the winner order is that child's list with
// a few entries of other children merged in.  The child, A, is the one that holds out longest,
// the one with the best entry (lk, lp) for the node's LAST visitor (not always the one with the
// best next entry: a child whose score is mostly exploration starts high and drops at once).
// Only a child whose next entry comes before the last-visitor entry (lk0, lp0) of the child
// with the best next entry can be A or get an entry in (A's last entry is at or before that
// one), so these few are listed one per lane first.  Every other child's entries that can get
// in come before (lk, lp); when there are at most 64 of them in all, each finds its place
// directly: the number of A's entries that come before it (a bisection on A's list, evaluated
// once into LDS) plus the number of such entries of other children that do.  No threshold
// search, no sort.  Exactness rests on: A's entries 0 .. m-1 in order (checked one by one);
// every other child's used entries in order and its first unused one either not before
// (lk, lp) (count_before brackets the count by two exact evaluations) or looked at and placed
// behind the m-th winner (checked).  Then the best head at any step is never one of the heads
// left out, and merging the lists by (key, position) is the serial order.
// On success: order[q] = (child << 21) | visit number for the m visitors, cnt[] the visits
// per child.  On failure nothing the caller relies on has changed (order[] is scratch).
template <int R, bool RAVE>
__device__ __forceinline__ bool sparse_merge(const SelectArgs &a, const NodeCtx &c, int lane, const Kids<R, RAVE> &k,
                                             int best0, uint32_t lk0, uint32_t lp0, int m, WaveLds<R> &lds,
                                             uint32_t *order, int (&cnt)[R], bool &pending) {
    constexpr int F = R * kWave;
    const uint32_t uvl = (uint32_t)a.vl;
    // ---- the children that matter, one per lane ----
    int n0 = 0;
    bool listed[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i = r * kWave + lane;
        uint32_t hk = k.k1[r], hp = (uint32_t)i;
        if (k.k2[r] > k.k1[r]) {
            hk = k.k2[r];
            hp = (uint32_t)(F + i);
        }
        listed[r] = hk != 0u && (i == best0 || comes_before(hk, hp, lk0, lp0));
        const uint64_t cm = __ballot(listed[r]);
        if (listed[r]) {
            const int cl = n0 + __popcll(cm & ((1ull << lane) - 1ull));
            if (cl < kSparseMax) {
                lds.st_j0[cl] = i;
                lds.st_n[cl] = k.n[r];
                lds.st_w[cl] = k.w[r];
                lds.st_p[cl] = k.p[r];
                lds.st_vl[cl] = k.vl[r];
                lds.st_q2[cl] = k.q2[r];
            }
        }
        n0 += __popcll(cm);
    }
    if (n0 < 2 || n0 > kSparseMax) return false;
    wave_sync_memory();
    int ci = -1, cn = 0, cvl = 0;
    float cw = 0.0f, cp = 0.0f, cq2 = 0.0f;
    uint32_t hk = 0u, hp = 0xFFFFFFFFu, zk = 0u, zp = 0xFFFFFFFFu;  // the child's next entry and its last-visitor entry
    if (lane < n0) {
        ci = lds.st_j0[lane];
        cn = lds.st_n[lane];
        cw = lds.st_w[lane];
        cp = lds.st_p[lane];
        cvl = lds.st_vl[lane];
        cq2 = lds.st_q2[lane];
        entry_key<R, RAVE>(cn, cw, cp, cvl, cq2, c.ep, uvl, 0, ci, hk, hp);
        entry_key<R, RAVE>(cn, cw, cp, cvl, cq2, c.ep, uvl, m - 1, ci, zk, zp);
    }
    // ---- A: the child that holds out longest ----
    uint32_t lk, lp;
    wave_best(zk, zp, lk, lp);
    if (lk == 0u) return false;
    const uint64_t am = __ballot(lane < n0 && zk == lk && zp == lp);
    if (am == 0ull) return false;
    const int a_lane = __ffsll((long long)am) - 1;
    const int a_child = __builtin_amdgcn_readlane(ci, a_lane);
    const int a_n = __builtin_amdgcn_readlane(cn, a_lane);
    const int a_vl = __builtin_amdgcn_readlane(cvl, a_lane);
    const float a_w = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cw), a_lane));
    const float a_p = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cp), a_lane));
    const float a_q2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cq2), a_lane));
    // ---- the others that can get an entry in: next entry before (lk, lp) ----
    const bool is_cand = lane < n0 && lane != a_lane && hk != 0u && comes_before(hk, hp, lk, lp);
    if (__ballot(is_cand) == 0ull) return false;
    {
        // Far too many entries by the estimates: leave before anything exact is paid for.  An entry
        // of a child gets in only if fewer than m entries come before it; the child's next entry has
        // r0 of A's entries before it, so its entry number t has at least r0 + t, and no more than
        // m - r0 of its entries can get in, however many come before (lk, lp) (two children whose
        // scores hardly move with virtual loss, a RAVE blend that dominates both, can have hundreds
        // there and still only meet at the very end).
        int est = 0;
        if (is_cand) {
            const int r0 = predict_count<RAVE>(a_n, a_w, a_p, a_vl, a_q2, c.ep, uvl, key_score(hk), m);
            const int room = m - r0 > 1 ? m - r0 : 1;
            est = predict_count<RAVE>(cn, cw, cp, cvl, cq2, c.ep, uvl, key_score(lk), kSparseMax + 1);
            est = est < room ? est : room;
        }
        // (a little below the capacity: the exact counts tend to come out above the estimates, and
        // a refusal after them costs three times what one here does)
        if (wave_sum_i32(est) > kSparseMax - 4) return false;
    }
    // ---- A's entries, all m of them, evaluated once into LDS and checked: none may come before its
    // predecessor (its head then stays at or before (lk, lp) throughout) ----
    // as one 64-bit number per entry, smaller = played earlier: inverted key above the position
    unsigned long long *akp = reinterpret_cast<unsigned long long *>(lds.key[0]);  // m < kHeavyMin = kBatchCap / 2 entries
    {
        bool bad_a = false;
        uint32_t carry_k = 0xFFFFFFFFu, carry_p = 0u;  // entry before the chunk
        for (int base = 0; base < m; base += kWave) {
            const int j = base + lane;
            uint32_t kk = 0u, pp = 0xFFFFFFFFu;
            if (j < m) {
                entry_key<R, RAVE>(a_n, a_w, a_p, a_vl, a_q2, c.ep, uvl, j, a_child, kk, pp);
                akp[j] = ((unsigned long long)~kk << 32) | pp;
            }
            uint32_t pk = (uint32_t)__shfl_up((int)kk, 1, kWave);
            uint32_t ppos = (uint32_t)__shfl_up((int)pp, 1, kWave);
            if (lane == 0) {
                pk = carry_k;
                ppos = carry_p;
            }
            if (j < m && (kk == 0u || comes_before(kk, pp, pk, ppos))) bad_a = true;
            carry_k = (uint32_t)__builtin_amdgcn_readlane((int)kk, 63);
            carry_p = (uint32_t)__builtin_amdgcn_readlane((int)pp, 63);
        }
        if (__ballot(bad_a) != 0ull) return false;
    }
    wave_sync_memory();
    // how many of A's entries come before the entry (tk, tp): the list is in order, so a bisection
    // on the exact keys
    auto rank_in_a = [&](uint32_t tk, uint32_t tp) {
        const unsigned long long t64 = ((unsigned long long)~tk << 32) | tp;
        int lo = 0, hi = m;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (akp[mid] < t64) lo = mid + 1;
            else hi = mid;
        }
        return lo;
    };
    // ---- how many entries each of the others has before (lk, lp), at most m - r0 (see above) ----
    int cc = 0, cap = 1;
    if (is_cand) {
        cap = m - rank_in_a(hk, hp);  // at least 1: A's last entry does not come before this one
        if (cap > kSparseMax + 1) cap = kSparseMax + 1;
        if (cap < 1) cap = 1;
        cc = count_before<R, RAVE>(cn, cw, cp, cvl, cq2, c.ep, uvl, ci, lk, lp, cap, true);
    }
    const int inc = wave_inclusive_sum(cc, lane);
    const int total = __builtin_amdgcn_readlane(inc, 63);
    if (total > kSparseMax) return false;
    const int start = inc - cc;
    // ---- one lane per entry: (lane of its child, visit number) ----
    for (int t = 0; t < cc; t++) lds.hist[start + t] = lane | (t << 8);  // start + cc <= total <= 64
    wave_sync_memory();
    int bad = 0;  // nonzero: the merge is refused
    uint32_t ek = 0u, epos = 0xFFFFFFFFu;
    int e_child = -1, e_t = 0, rank_a = m;
    if (lane < total) {
        const uint32_t w0 = (uint32_t)lds.hist[lane];
        const int e_cl = (int)(w0 & 255u);
        e_t = (int)(w0 >> 8);
        e_child = lds.st_j0[e_cl];
        entry_key<R, RAVE>(lds.st_n[e_cl], lds.st_w[e_cl], lds.st_p[e_cl], lds.st_vl[e_cl], lds.st_q2[e_cl], c.ep, uvl,
                           e_t, e_child, ek, epos);
        if (ek == 0u) bad = 1;
        rank_a = rank_in_a(ek, epos);
    }
    {
        // a child's entries sit in neighbouring lanes, in visit order: none may come before its predecessor
        const uint32_t pk = (uint32_t)__shfl_up((int)ek, 1, kWave);
        const uint32_t pp = (uint32_t)__shfl_up((int)epos, 1, kWave);
        if (lane < total && e_t > 0 && comes_before(ek, epos, pk, pp)) bad = 2;
    }
    // ---- the other entries before each of them (equal keys at one position: one child, visit order) ----
    // as 64-bit numbers again, with the lane below the position: all different, a child's entries in visit order
    unsigned long long *ekp = reinterpret_cast<unsigned long long *>(lds.key[1]);  // all lanes read all entries: through LDS
    const unsigned long long e64 =
        lane < total ? ((unsigned long long)~ek << 32) | ((unsigned long long)epos << 8) | (unsigned)lane : ~0ull;
    ekp[lane] = e64;
    wave_sync_memory();
    int fr = 0;
    // (eight reads in flight at a time: one wavefront alone waits out every LDS access it depends on)
    for (int e0 = 0; e0 < total; e0 += 8) {
        unsigned long long o[8];
#pragma unroll
        for (int u = 0; u < 8; u++) o[u] = ekp[e0 + u];  // lanes past `total` hold the largest number: before nothing
#pragma unroll
        for (int u = 0; u < 8; u++) fr += o[u] < e64 ? 1 : 0;
    }
    const int posn = rank_a + fr;
    const bool valid = lane < total && posn < m;
    {
        // of a child's entries the ones that get in are the first ones
        const int pv = __shfl_up(valid ? 1 : 0, 1, kWave);
        if (valid && e_t > 0 && pv == 0) bad = 3;
    }
    const uint64_t vmask = __ballot(valid);
    const int nfv = __popcll(vmask);
    int mine_in = 0;  // entries of this lane's child that get in
    if (is_cand) {
        const uint64_t mine = cc >= 64 ? ~0ull : ((1ull << cc) - 1ull);
        mine_in = __popcll((vmask >> start) & mine);
        // a child all of whose counted entries get in, counted up to its limit: its next entry was
        // not looked at
        if (mine_in == cc && cc == cap) bad = 4;
    }
    {
        const int why = (int)wave_max_u32((uint32_t)bad);
        if (why != 0) return false;
    }
    // ---- the winner order: the others' entries at their places, A's in between ----
    close_pending(pending);  // the previous node's partition may still read the order buffer
    for (int q = lane; q < m; q += kWave) order[q] = 0u;
    wave_sync_memory();
    if (valid) order[posn] = 0x80000000u | ((uint32_t)e_child << 21) | (uint32_t)e_t;
    wave_sync_memory();
    int seen = 0;
    for (int base = 0; base < m; base += kWave) {
        const int q = base + lane;
        const uint32_t v = q < m ? order[q] : 0u;
        const bool other = (v >> 31) != 0u;
        const uint64_t om = __ballot(other);
        const int below = seen + __popcll(om & ((1ull << lane) - 1ull));
        if (q < m) order[q] = other ? (v & 0x7FFFFFFFu) : (((uint32_t)a_child << 21) | (uint32_t)(q - below));
        seen += __popcll(om);
    }
    if (seen != nfv) return false;  // two entries at one place: cannot happen when the checks hold
    // ---- visits per child, back to the lanes that hold the children ----
    if (lane < n0) lds.hist[kSparseMax + lane] = lane == a_lane ? m - nfv : mine_in;
    wave_sync_memory();
    int cl_run = 0;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint64_t cm = __ballot(listed[r]);
        cnt[r] = listed[r] ? lds.hist[kSparseMax + cl_run + __popcll(cm & ((1ull << lane) - 1ull))] : 0;
        cl_run += __popcll(cm);
    }
    return true;
}


// A wide node (more than 64 child slots) whose visitors split, settled as a narrow one.  Of all its
// children only those can be chosen whose next entry comes before the entry (lk0, lp0) that the child
// with the best next entry, B, shows its LAST visitor, provided B's entries are in order: B's head is
// then at or before (lk0, lp0) at every step, so a child whose head does not come before that entry is
// never the best.  Where B's order is provable (keys_provably_monotone) and these children are at most
// 64, they are moved to one lane each, in child order (positions keep their order, and every first-scan
// candidate still comes before every second-scan one), and the water level of the narrow class settles
// them: its probes walk one round of children instead of R.  The winner order comes back with the
// children's own indices, the visits per child to the lanes that hold them.  Returns false with nothing
// the caller relies on changed (cnt[] zero).
template <int R, bool RAVE>
__device__ __forceinline__ bool narrow_water_level(const SelectArgs &a, const NodeCtx &c, int lane,
                                                   const Kids<R, RAVE> &k, int soff, int best0, uint32_t lk0,
                                                   uint32_t lp0, int m, WaveLds<R> &lds, int (&cnt)[R], int &lds_cur,
                                                   uint32_t *order, bool &pending) {
    static_assert(R > 1, "a narrow node is settled as it is");
    constexpr int F = R * kWave;
    const uint32_t uvl = (uint32_t)a.vl;
    int n0 = 0;
    bool listed[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i = r * kWave + lane;
        uint32_t hk = k.k1[r], hp = (uint32_t)i;
        if (k.k2[r] > k.k1[r]) {
            hk = k.k2[r];
            hp = (uint32_t)(F + i);
        }
        listed[r] = hk != 0u && (i == best0 || comes_before(hk, hp, lk0, lp0));
        const uint64_t cm = __ballot(listed[r]);
        if (listed[r]) {
            const int cl = n0 + __popcll(cm & ((1ull << lane) - 1ull));
            if (cl < kWave) {
                lds.st_j0[cl] = i;
                lds.st_n[cl] = k.n[r];
                lds.st_w[cl] = k.w[r];
                lds.st_p[cl] = k.p[r];
                lds.st_vl[cl] = k.vl[r];
                lds.st_q2[cl] = k.q2[r];
            }
        }
        n0 += __popcll(cm);
    }
    if (n0 < 2 || n0 > kWave) return false;
    wave_sync_memory();
    Kids<1, RAVE> kc;
    int orig = -1;
    kc.part[0] = lane < n0;
    kc.n[0] = 0;
    kc.w[0] = 0.0f;
    kc.p[0] = 0.0f;
    kc.vl[0] = 0;
    kc.q2[0] = 0.0f;
    if (lane < n0) {
        orig = lds.st_j0[lane];
        kc.n[0] = lds.st_n[lane];
        kc.w[0] = lds.st_w[lane];
        kc.p[0] = lds.st_p[lane];
        kc.vl[0] = lds.st_vl[lane];
        kc.q2[0] = lds.st_q2[lane];
    }
    score_round<1, RAVE>(kc, 0, c.ep);
    {
        const bool b_ok = orig == best0 && keys_provably_monotone<RAVE>(kc.n[0], kc.w[0], kc.p[0], kc.vl[0], kc.q2[0],
                                                                       c.ep, uvl, m - 1);
        if (__ballot(b_ok) == 0ull) return false;
    }
    wave_sync_memory();  // every lane has read its child: the scratch changes hands
    WaveLds<1> &l1 = reinterpret_cast<WaveLds<1> &>(lds);
    NodeCtx c1 = c;
    c1.cc = n0;
    c1.nelig = n0;
    int cnt1[1] = {0};
    const int zero1[1] = {0};
    int cur = -1;
    if (!water_level<1, RAVE>(a, c1, lane, kc, soff, 0, m, zero1, l1, cnt1, true, cur, false, zero1, order, pending))
        return false;
    // ---- back to the node's own child indices ----
    // (every lane takes part in the exchange, whether it has an entry in this pass or not)
    if (cur >= 0) {
        for (int base = 0; base < m; base += kWave) {
            const int q = base + lane;
            const uint32_t v = q < m ? order[q] : 0u;
            const int i = __shfl(orig, (int)((v >> 21) & 63u), kWave);
            if (q < m) order[q] = (v & 0x80000000u) | ((uint32_t)i << 21) | (v & 0x1FFFFFu);
        }
    } else {
        for (int base = 0; base < m; base += kWave) {
            const int q = base + lane;
            const int cl = q < m ? a.sc_child[soff + q] : 0;
            const int i = __shfl(orig, cl & 63, kWave);
            if (q < m) a.sc_child[soff + q] = i;
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) lds.st_j0[r * kWave + lane] = 0;
    wave_sync_memory();
    if (lane < n0) lds.st_j0[orig] = cnt1[0];
    wave_sync_memory();
#pragma unroll
    for (int r = 0; r < R; r++) cnt[r] = lds.st_j0[r * kWave + lane];
    lds_cur = cur;
    wave_sync_memory();
    return true;
}

// ---- Chains of nodes whose visitors all follow one child ----
// Most crowded nodes below the top of a tree are of that kind, often a dozen in a row (a whole
// selection of the Go workload with 16 visitors per tree starts with a chain of them), and on such a
// node nothing is decided: the visitors stay together, in the same order.  When the owner finds such a
// node (single_run), it does not share out its visitors: it hands the node's child to its three helpers,
// which walk down from there in lockstep for as long as the visitors stay together (chain_walk): each
// loads and scores its rounds of the children (statistics, legality bits and the child ranges of all
// children in range in ONE trip to memory), leaves its best candidate, the best candidate of its other
// children and the best child's statistics in LDS; after one block barrier each of them knows the
// node's best child and the best candidate of all others, makes the one-winner test of single_run
// (the entry the best child shows the LAST visitor still comes first, and its entries are in order)
// and moves on into the child.  One barrier and one dependent trip to memory per level, no partition:
// the visitor list does not change, so the walk does not even read it; it records the children it
// took, and when it has stopped the three write the visitors' path entries for all its levels at
// once, the level of the owner's node included, and the list into the buffer the next node reads
// (chain_finish).  The walk stops at a leaf (or the depth cap), or at the first node that fails the
// test: that node's children, loaded and scored, are left in the LDS scratch together with the
// verdict, and select_group settles it from there.  The owner takes the walk's barriers with it
// (a block barrier counts every wavefront) and does nothing else meanwhile: the code of the walk
// stays out of the owner's own, whose registers are its scarcest resource.
// One round of a node's children, as select_group collects them from the LDS scratch of fan-out class R.
template <int R>
__device__ __forceinline__ void chain_dump(LdsBytesP base, int i, int n, float w, float p, int vl, float q2,
                                           uint32_t k1, uint32_t k2, bool part) {
    typedef __attribute__((address_space(3))) WaveLds<R> *P;
    P l = (P)base;
    l->st_n[i] = n;
    l->st_w[i] = w;
    l->st_p[i] = p;
    l->st_vl[i] = vl;
    l->st_q2[i] = q2;
    l->key[0][i] = k1;
    l->key[1][i] = k2;
    l->pay[i] = part ? 1u : 0u;
}

// The kernel's arguments where the hardware put them: a function that is not inlined reads what it needs
// from there (scalar loads through the constant cache) instead of receiving copies through the stack,
// which cost a round trip to memory at every call.
struct SelectKernArgs {
    ForestDev f;
    SelectArgs a;
};
typedef const __attribute__((address_space(4))) SelectKernArgs *KernArgsP;
static_assert(offsetof(SelectKernArgs, a) == sizeof(ForestDev),
              "k_select_groups(ForestDev, SelectArgs): the second argument follows the first");

// What one of the walking wavefronts found among the children it loaded, one level.
struct ChainSlot {
    uint32_t bk, bpos;  // its best candidate (key 0 = none)
    uint32_t sk, spos;  // the best candidate of its children other than that one's child
    int n, vl;          // that child's statistics and child range
    float w, p, q2;
    int sx, sy;
    uint32_t any1;      // one of its children has a real first-scan key
};
constexpr int kChainWalkers = 3;
__shared__ ChainSlot g_chain_slot[2][kChainWalkers];

// wi: which of the three walking wavefronts this is.  Every block barrier in here is also taken by the owner,
// which waits the walk out (owner_loop).
// The statistics of the children one walking wavefront is responsible for, as loaded.
template <int Q>
struct ChainKids {
    int n[Q], vl[Q];
    float w[Q], p[Q], q2[Q];
    int2 sp[Q];
    uint32_t word[Q];  // legality bits
};

template <int RMAX, bool RAVE>
__device__ __noinline__ int chain_walk(KernArgsP ka, LdsBytesP scratch, int wi, int lane, int node, int np, int cb,
                                       int cc, int depth, int m) {
    constexpr int F = RMAX * kWave;
    // a layout without wide nodes: one wavefront walks alone (no exchange, no barrier per level)
    constexpr bool SOLO = RMAX == 1;
    constexpr int Q = SOLO ? 1 : (RMAX + kChainWalkers - 1) / kChainWalkers;  // rounds of children per wavefront: wi*Q .. wi*Q+Q-1
    const int32_t *const fN = ka->f.N, *const fVL = ka->f.VL;
    const float *const fW = ka->f.W, *const fP = ka->f.P, *const fq2 = ka->f.q2;
    const uint32_t *const flegal = ka->f.legal;
    const int2 *const fspan = ka->f.span;
    const int max_depth = ka->a.max_depth, pw = ka->a.pw;
    const float c_puct = ka->a.c_puct;
    const uint32_t uvl = (uint32_t)ka->a.vl;
    long long *const trace = ka->a.trace;
    int level = 1;  // level 0 is the node settled before, whose child this walk starts at
    int bars = 0;   // block barriers taken
    int kids = 0, contested = 0, best0 = -1, second = 0;
    uint32_t lk0 = 0u;
    auto eligible = [&](int np_, int cc_) {
        int e = cc_;
        if (pw) {
            const int kk = ceil_sqrt_i32(np_);
            e = kk < cc_ ? kk : cc_;
        }
        return e;
    };
    // asks for this wavefront's rounds of the children cb_ .. cb_ + nelig_ - 1 (nothing waits for them here)
    auto issue = [&](ChainKids<Q> &k, int cb_, int nelig_) {
#pragma unroll
        for (int q = 0; q < Q; q++) {
            const int r = wi * Q + q;
            const int i = r * kWave + lane;
            const bool in = i < nelig_;
            const int id = cb_ + i;
            k.word[q] = 0xFFFFFFFFu;
            k.n[q] = 0;
            k.w[q] = 0.0f;
            k.p[q] = 0.0f;
            k.vl[q] = 0;
            k.q2[q] = 0.0f;
            k.sp[q] = int2{0, 0};
            if (r * kWave < nelig_) {  // uniform: rounds the node lacks are skipped
                if (in && flegal) k.word[q] = flegal[(uint32_t)id >> 5];
                if (in) {
                    k.n[q] = fN[id];
                    k.w[q] = fW[id];
                    k.p[q] = fP[id];
                    k.vl[q] = fVL[id];
                    if (RAVE) k.q2[q] = fq2[id];
                    k.sp[q] = fspan[id];
                }
            }
        }
    };
    int nelig = eligible(np, cc);
    bool alive = !(cc <= 0 || depth >= max_depth || level >= kChainMaxLevels);
    ChainKids<Q> kids_a, kids_b;
    if (alive) issue(kids_a, cb, nelig);
    // One level: `cur` holds (or is about to receive) the children of the node the walk stands at; the
    // children of the child it moves on into are asked for into `nxt` as soon as that child is known, before
    // the one-winner test, whose arithmetic then runs while they are on their way (they are dropped if the
    // test fails).  Returns whether the walk goes on.
    auto step = [&](ChainKids<Q> &cur, ChainKids<Q> &nxt) -> bool {
        const long long tr0 = trace && wi == 0 ? wall_clock64() : 0ll;
        const float ep = c_puct * sqrtf((float)np);
        const int par = level & 1;
        int (&kn)[Q] = cur.n;
        int (&kvl)[Q] = cur.vl;
        float (&kw)[Q] = cur.w;
        float (&kp)[Q] = cur.p;
        float (&kq2)[Q] = cur.q2;
        int2 (&ksp)[Q] = cur.sp;
        uint32_t k1[Q], k2[Q];
        bool kin[Q];
#pragma unroll
        for (int q = 0; q < Q; q++) {
            const int r = wi * Q + q;
            const int i = r * kWave + lane;
            const int id = cb + i;
            kin[q] = i < nelig && ((cur.word[q] >> ((uint32_t)id & 31u)) & 1u);
            k1[q] = k2[q] = 0u;
            if (r * kWave < nelig) {
                if (kin[q]) {
                    child_keys<RAVE>(kn[q], kw[q], kp[q], kvl[q], kq2[q], ep, k1[q], k2[q]);
                } else {
                    kn[q] = 0;
                    kw[q] = 0.0f;
                    kp[q] = 0.0f;
                    kvl[q] = 0;
                    kq2[q] = 0.0f;
                }
            }
        }
        // ---- its best candidate, and the best candidate of its other children ----
        uint32_t bk = 0u, bpos = 0xFFFFFFFFu;
        bool has1 = false, odd1 = false;
#pragma unroll
        for (int q = 0; q < Q; q++) {
            has1 |= k1[q] != 0u;
            if (RAVE) odd1 |= kin[q] && !(fabsf(kw[q]) <= 3.0e38f);
            if (k1[q] > bk) { bk = k1[q]; bpos = (uint32_t)((wi * Q + q) * kWave + lane); }
        }
#pragma unroll
        for (int q = 0; q < Q; q++)
            if (k2[q] > bk) { bk = k2[q]; bpos = (uint32_t)(F + (wi * Q + q) * kWave + lane); }
        uint32_t hk, hp;
        wave_best(bk, bpos, hk, hp);
        const uint32_t mine = hk == 0u ? 0xFFFFFFFFu : (hp >= (uint32_t)F ? hp - (uint32_t)F : hp);
        uint32_t ok_ = 0u, opos = 0xFFFFFFFFu;
#pragma unroll
        for (int q = 0; q < Q; q++) {
            const uint32_t i = (uint32_t)((wi * Q + q) * kWave + lane);
            if (i != mine && k1[q] > ok_) { ok_ = k1[q]; opos = i; }
        }
#pragma unroll
        for (int q = 0; q < Q; q++) {
            const uint32_t i = (uint32_t)((wi * Q + q) * kWave + lane);
            if (i != mine && k2[q] > ok_) { ok_ = k2[q]; opos = (uint32_t)F + i; }
        }
        uint32_t sk, spos;
        wave_best(ok_, opos, sk, spos);
        int bn, bvl, bsx, bsy;
        float bw, bp, bq2;
        bool any1, odd_any = false;
        if (SOLO) {
            int tn = kn[0], tvl = kvl[0], tsx = ksp[0].x, tsy = ksp[0].y;
            float tw = kw[0], tp = kp[0], tq2 = kq2[0];
            const int ml = (int)(mine & 63u);
            bn = __builtin_amdgcn_readlane(tn, ml);
            bvl = __builtin_amdgcn_readlane(tvl, ml);
            bsx = __builtin_amdgcn_readlane(tsx, ml);
            bsy = __builtin_amdgcn_readlane(tsy, ml);
            bw = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tw), ml));
            bp = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tp), ml));
            bq2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tq2), ml));
            any1 = __ballot(has1) != 0ull;
            if (RAVE) odd_any = __ballot(odd1) != 0ull;
        } else {
        {
            int tn = 0, tvl = 0, tsx = 0, tsy = 0;
            float tw = 0.0f, tp = 0.0f, tq2 = 0.0f;
#pragma unroll
            for (int q = 0; q < Q; q++) {
                if ((uint32_t)(wi * Q + q) == (mine >> 6)) {
                    tn = kn[q];
                    tw = kw[q];
                    tp = kp[q];
                    tvl = kvl[q];
                    tq2 = kq2[q];
                    tsx = ksp[q].x;
                    tsy = ksp[q].y;
                }
            }
            // the lane that holds the wavefront's best child writes the slot (one lane, one pass)
            const bool any1w = __ballot(has1) != 0ull;
            const bool odd1w = RAVE && __ballot(odd1) != 0ull;
            if (lane == (int)(mine == 0xFFFFFFFFu ? 0u : (mine & 63u))) {
                ChainSlot &sl = g_chain_slot[par][wi];
                sl.bk = hk;
                sl.bpos = hp;
                sl.sk = sk;
                sl.spos = spos;
                sl.n = tn;
                sl.vl = tvl;
                sl.w = tw;
                sl.p = tp;
                sl.q2 = tq2;
                sl.sx = tsx;
                sl.sy = tsy;
                sl.any1 = (any1w ? 1u : 0u) | (odd1w ? 2u : 0u);
            }
        }
        __syncthreads();
        bars++;
        // ---- the same over the three wavefronts ----
        hk = 0u;
        hp = 0xFFFFFFFFu;
        int won = 0;
        uint32_t a1 = 0u;
#pragma unroll
        for (int w = 0; w < kChainWalkers; w++) {
            const uint32_t k_ = g_chain_slot[par][w].bk, p_ = g_chain_slot[par][w].bpos;
            a1 |= g_chain_slot[par][w].any1;
            if (k_ != 0u && comes_before(k_, p_, hk, hp)) {
                hk = k_;
                hp = p_;
                won = w;
            }
        }
        won = __builtin_amdgcn_readfirstlane(won);
        sk = 0u;
        spos = 0xFFFFFFFFu;
#pragma unroll
        for (int w = 0; w < kChainWalkers; w++) {
            const uint32_t k_ = w == won ? g_chain_slot[par][w].sk : g_chain_slot[par][w].bk;
            const uint32_t p_ = w == won ? g_chain_slot[par][w].spos : g_chain_slot[par][w].bpos;
            if (k_ != 0u && comes_before(k_, p_, sk, spos)) {
                sk = k_;
                spos = p_;
            }
        }
        const ChainSlot &ws = g_chain_slot[par][won];
        bn = __builtin_amdgcn_readfirstlane(ws.n);
        bvl = __builtin_amdgcn_readfirstlane(ws.vl);
        bsx = __builtin_amdgcn_readfirstlane(ws.sx);
        bsy = __builtin_amdgcn_readfirstlane(ws.sy);
        bw = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(ws.w)));
        bp = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(ws.p)));
        bq2 = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(ws.q2)));
        hk = (uint32_t)__builtin_amdgcn_readfirstlane((int)hk);
        hp = (uint32_t)__builtin_amdgcn_readfirstlane((int)hp);
        sk = (uint32_t)__builtin_amdgcn_readfirstlane((int)sk);
        spos = (uint32_t)__builtin_amdgcn_readfirstlane((int)spos);
        any1 = (__builtin_amdgcn_readfirstlane((int)a1) & 1) != 0;
        odd_any = (__builtin_amdgcn_readfirstlane((int)a1) & 2) != 0;
        }  // !SOLO
        // ---- the children of the child the walk would move on into: on their way during the test ----
        const int n_nelig = eligible(bn, bsy);
        const bool n_alive = hk != 0u && !(bsy <= 0 || depth + 1 >= max_depth || level + 1 >= kChainMaxLevels);
        if (n_alive) issue(nxt, bsx, n_nelig);
        // ---- the one-winner test (single_run) ----
        // (with RAVE and no real first-scan score at all the reference never runs its second scan;
        // select_group knows, and gets no verdict)
        // (a child whose value sum is not finite: the node is settled one visitor after the other, select_group)
        bool one = hk != 0u && (!RAVE || (any1 && !odd_any));
        const int best = (int)(hp >= (uint32_t)F ? hp - (uint32_t)F : hp);
        if (one) {
            uint32_t lk, lp;
            entry_key<RMAX, RAVE>(bn, bw, bp, bvl, bq2, ep, uvl, m - 1, best, lk, lp);
            if (lk == 0u) {
                one = false;
            } else if (sk != 0u && !comes_before(lk, lp, sk, spos)) {
                one = false;
                contested = 1;
                best0 = best;
                lk0 = lk;
                second = lp >= (uint32_t)F ? 1 : 0;
            } else if (!entries_in_order<RMAX, RAVE>(bn, bw, bp, bvl, bq2, ep, uvl, best, m, lane)) {
                one = false;
            }
        }
        if (!one) {
            // the node's children, where select_group collects them (its own fan-out class)
            kids = 1;
            if (cc <= kWave) {
#pragma unroll
                for (int q = 0; q < Q; q++)
                    if (wi * Q + q < 1)
                        chain_dump<1>(scratch, lane, kn[q], kw[q], kp[q], kvl[q], kq2[q], k1[q], k2[q], kin[q]);
            } else {
#pragma unroll
                for (int q = 0; q < Q; q++)
                    if (wi * Q + q < RMAX)
                        chain_dump<RMAX>(scratch, (wi * Q + q) * kWave + lane, kn[q], kw[q], kp[q], kvl[q], kq2[q], k1[q],
                                         k2[q], kin[q]);
            }
            return false;
        }
        // ---- every visitor takes that child ----
        const int child = cb + best;
        if (lane == 0) g_chain.nodes[level] = child;  // every walker for itself: chain_finish reads them without a barrier
        if (wi == 0 && lane == 0) {
            atomicAdd(ka->f.VL + child, (int)(uvl * (uint32_t)m));
            int32_t *const stats = ka->a.stats;
            if (stats) {
                atomicAdd(stats + 0, 1);
                atomicAdd(stats + 1, 1);
                atomicAdd(stats + 2, m);
            }
            if (trace) {
                const int ti = atomicAdd(ka->a.trace_n, 1);
                if (ti < ka->a.trace_cap) {
                    trace[12 * ti + 0] = tr0;
                    trace[12 * ti + 1] = wall_clock64();
                    trace[12 * ti + 2] = (long long)m | ((long long)depth << 32) | (5ll << 60);
                    trace[12 * ti + 3] = (long long)node;
                    for (int q = 0; q < 8; q++) trace[12 * ti + 4 + q] = 0;
                }
            }
        }
        node = child;
        np = bn;
        cb = bsx;
        cc = bsy;
        depth++;
        level++;
        nelig = n_nelig;
        alive = n_alive;
        return n_alive;
    };
    if (alive) {
        for (;;) {
            if (!step(kids_a, kids_b)) break;
            if (!step(kids_b, kids_a)) break;
        }
    }
    if (wi == 0 && lane == 0) {
        g_chain.levels = level;
        g_chain.e_node = node;
        g_chain.e_np = np;
        g_chain.e_cb = cb;
        g_chain.e_cc = cc;
        g_chain.e_depth = depth;
        g_chain.e_kids = kids;
        g_chain.e_contested = contested;
        g_chain.e_best0 = best0;
        g_chain.e_lk0 = lk0;
        g_chain.e_second = second;
        // the owner counts the block barriers it takes with the walk: it leaves after the one that follows these
        g_chain.n_barriers = bars;
    }
    return level;
}

// After a walk: the path entries of its visitors for every level, the first of which is the node settled
// before the walk (all of whose visitors went into the child the walk started at, in their order), and
// their list where the node the walk stopped at reads it.  Shared by the three wavefronts.
__device__ __noinline__ void chain_finish(KernArgsP ka, int tid3, int n_threads, int k, int d0, int off, int m) {
    const int32_t *src = d0 == 0 ? ka->a.seg0 : ka->a.seg[(d0 - 1) & 1];
    int32_t *dst = ka->a.seg[(d0 + k - 1) & 1];
    int32_t *paths = ka->a.paths;
    const int stride = ka->a.stride;
    for (int j = tid3; j < m; j += n_threads) {
        const int t = src[off + j];
        for (int i = 0; i < k; i++) paths[(size_t)(d0 + 1 + i) * stride + t] = g_chain.nodes[i];
        if (dst != src) dst[off + j] = t;
    }
}

// Where the walk goes on after a multi-visitor node whose visitors all chose one child.
// Called by one slice of a heavy node once it knows a lower bound of every child's visitors (low[]: the child's
// entries among the first ranks of the node's winner order; at most `slack` more visitors can come).  A child
// that is sure to get kHeavyMin visitors will be cut into slices of S = slice_size(its visitors), and boundary
// b of it (rank b * S) depends on the child's own statistics only, which nothing changes before the child
// itself is shared out.  So the boundaries that are sure to lie within the child's visitors, whatever the final
// count, become items of the work queue right away (kind 4: pad[1] the child's context, pad[2] = b | S << 8),
// taken by wavefronts that would otherwise wait; the child's slices find them in the boundary table.  The
// child's context is handed out here and left in the node's context ([16 + kHeavyFanout + i] = context + 1, 0 =
// none; [5] = the number of the select call once that is written), where the wavefront that publishes the child
// picks it up.  Nothing here is a guess: a boundary that turns out not to be needed (the child is settled
// otherwise) is a wasted computation, never a wrong one.
template <int R, bool RAVE>
__device__ __forceinline__ void prefetch_boundaries(const ForestDev &f, const SelectArgs &a, const NodeCtx &c, int lane,
                                                    const Kids<R, RAVE> &k, const int (&low)[R], int slack, int depth,
                                                    int *ctx) {
    int nb[R], sz[R], cid[R];
    int mine = 0;
#pragma unroll
    for (int r = 0; r < R; r++) {
        nb[r] = 0;
        sz[r] = 0;
        cid[r] = -1;
        const int L = low[r];
        if (L >= kHeavyMin && r * kWave + lane < c.nelig) {
            const int S = slice_size(L);
            if (S == slice_size(L + slack) && f.span[c.cb + r * kWave + lane].y > 0) {
                // every boundary the child can need, whatever its final count: the one behind its last slice
                // included (a boundary does not depend on the count; one too many is a wasted computation)
                int n = (L + slack + S - 1) / S;
                n = n < kMaxSlices ? n : kMaxSlices;
                if (n >= 1) {
                    const int id = atomicAdd(a.hctx_n, 1);
                    if (id < a.hctx_cap) {
                        nb[r] = n;
                        sz[r] = S;
                        cid[r] = id;
                        mine += n;
                    }
                }
            }
        }
    }
    const int inc = wave_inclusive_sum(mine, lane);
    const int total = __builtin_amdgcn_readlane(inc, 63);
    int slot0 = 0;
    if (total > 0) {
        if (lane == 0) slot0 = atomicAdd(a.sched_tail, total);
        slot0 = __builtin_amdgcn_readfirstlane(slot0);
        if (slot0 + total > a.q_cap) {
            if (lane == 0) atomicExch(a.sched_wait + 1, 2);  // queue overflow: cannot happen on a tree
            return;
        }
    }
    int at = slot0 + inc - mine;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i = r * kWave + lane;
        ctx[16 + kHeavyFanout + i] = cid[r] + 1;
        for (int b = 1; b <= nb[r]; b++) {
            Item it;
            it.node = c.cb + i;
            it.off = 0;
            it.m = low[r];
            it.np = k.n[r];
            it.depth = depth + 1;
            it.pad[0] = 4;
            it.pad[1] = cid[r];
            it.pad[2] = b | (sz[r] << 8);
            a.items_q[at + b - 1] = it;
        }
        at += nb[r];
    }
    if (lane == 0) ctx[5] = a.epoch;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    at = slot0 + inc - mine;
    for (int j = 0; j < mine; j++)
        __hip_atomic_store(a.q_ready + at + j, a.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct Continuation {
    int node;
    int off;
    int m;
    int np;
    int2 span;  // (child_begin, child_count) of that node, loaded ahead of time
    bool ahead;  // two helpers load their share of that node's children (load_ahead), if it is a wide one
    bool chain_open;  // the request that shares out this node's visitors also starts the walk at that node (chain_walk)
};

// All visitors of a multi-visitor item.  Records the chosen child of every visitor, bumps
// virtual loss, partitions the visitors by child into seg_out, writes the next path
// entry; the largest part stays with this wavefront (next), the other parts with several
// visitors become items of the work queue, children with one visitor go to the
// single-visitor queue.  Returns kStepLeaf when no child takes part in the selection.
//
// A heavy node (kHeavyMin visitors or more) is cut into slices of its winner order, one
// queue item each, that wavefronts settle side by side: slice s covers the ranks between
// two boundaries, s and s+1, each a score threshold with the exact entry counts of every child
// above it (threshold_counts; a boundary may lie inside a pile of entries of one key).  Slice s
// works out boundary s+1 and leaves it in the node's boundary table, where slice s+1 picks it up:
// the two neighbours use the same numbers.  A slice starts the batch loop from the state "child i
// has had count_i(boundary s) visits" and must arrive exactly at count_i(boundary s+1); with that
// check, T_s >= T_s+1, and the batch loop's own checks, slice after slice starts from the true
// serial state, so the slices together are the serial order.  The slice that reaches the last visitor writes the visits per child; the
// wavefront that finishes last (a counter in the node's context) partitions the visitors
// and walks on, every other returns kStepParked.  Any failed check sends the whole node
// back to the one-wavefront path.
template <int R, bool RAVE, int RMAX>
__device__ __forceinline__ int select_group(const ForestDev &f, const SelectArgs &a, const NodeCtx &c, int lane,
                                            const Item &item, const int32_t *seg_in, int32_t *seg_out,
                                            WaveLds<R> &lds, PartLds<RMAX> &pl, bool &pending, Continuation &next,
                                            int preload) {
    // preload: 0 the children are loaded here; 1 two helpers are loading their share (load_ahead); 2 a walk down
    // one-winner nodes stopped at this node and left its children, scored, in the LDS scratch, with the verdict
    bool ahead = preload == 1;
    const int off = item.off, m = item.m, depth = item.depth;
    // a heavy node is settled and shared out by several wavefronts, which read its visitor
    // list: it must be complete before any of them is called in
    // where this node's winner order goes in sc_child / sc_occ when it does not fit LDS: the
    // two halves alternate with the depth, because the children of a heavy node are at work
    // while wavefronts still read the order of their parent
    const int soff = off + (depth & 1) * a.stride;
    // the visitor list of an item of kind 3, and of the slices of one, may not be there yet:
    // whoever shares out the visitors waits for it (below), settling them does not need it
    bool list_ok = !(item.pad[0] == 3 || (item.pad[0] == 1 && ((item.pad[2] >> 30) & 1)));
    if (m >= kHeavyMin) close_pending(pending);
    Kids<R, RAVE> k;
    int cnt[R];
    uint32_t bk = 0u, bpos = 0xFFFFFFFFu;
    if (item.pad[0] == 2) {
        // a part of a heavy node's partition: of the children only the visit counts are needed
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int i = r * kWave + lane;
            k.n[r] = i < c.nelig ? f.N[c.cb + i] : 0;
            k.w[r] = k.p[r] = k.q2[r] = 0.0f;
            k.vl[r] = 0;
            k.k1[r] = k.k2[r] = 0u;
            k.part[r] = false;
            cnt[r] = 0;
        }
    } else {
        if (preload == 2) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                const int i = r * kWave + lane;
                k.n[r] = lds.st_n[i];
                k.w[r] = lds.st_w[i];
                k.p[r] = lds.st_p[i];
                k.vl[r] = lds.st_vl[i];
                k.q2[r] = lds.st_q2[i];
                k.k1[r] = lds.key[0][i];
                k.k2[r] = lds.key[1][i];
                k.part[r] = lds.pay[i] != 0u;
                cnt[r] = 0;
            }
        } else if (R > 1 && R == RMAX && !ahead) {
            // a wide node from the queue: the helpers are idle (or finish the partition of the node this
            // wavefront settled last), two of them take their share of the children
            close_pending(pending);
            if (lane == 0) {
                TeamCmd &cm = lds.cmd;
                cm.op = kOpLoad;
                cm.rounds = R;
                cm.pre_node = item.node;
                cm.pre_np = item.np;
                cm.pre_cb = c.cb;
                cm.pre_cc = c.cc;
            }
            __syncthreads();  // the request is open until close_pending
            pending = true;
            ahead = true;
        }
        if (preload == 2) {
        } else if (R > 1 && R == RMAX && ahead) {
            // this wavefront's share of the children; the rest is in LDS once the request is closed
            constexpr int S = AheadShare<R>::kRounds;
            load_score_rounds<R, RAVE, 0, (S < R ? S : R)>(f, c.cb, c.nelig, lane, a.rave_k, c.ep, k);
            close_pending(pending);
#pragma unroll
            for (int r = S; r < R; r++) {
                const int i = r * kWave + lane;
                k.n[r] = lds.st_n[i];
                k.w[r] = lds.st_w[i];
                k.p[r] = lds.st_p[i];
                k.vl[r] = lds.st_vl[i];
                k.q2[r] = lds.st_q2[i];
                k.k1[r] = lds.key[0][i];
                k.k2[r] = lds.key[1][i];
                k.part[r] = lds.pay[i] != 0u;
            }
#pragma unroll
            for (int r = 0; r < R; r++) cnt[r] = 0;
        } else {
            load_kids<R, RAVE, true>(f, c.cb, c.nelig, lane, a.rave_k, k);
#pragma unroll
            for (int r = 0; r < R; r++) {
                score_round<R, RAVE>(k, r, c.ep);
                cnt[r] = 0;
            }
        }
        if (RAVE) {
            // no real score in the first scan: the reference never runs the second one
            // (mcts_node.cpp:173-184); without keys every parallel path declines and the visitors
            // are played one at a time, where wave_pick applies the same rule
            bool any1 = false;
#pragma unroll
            for (int r = 0; r < R; r++) any1 |= k.k1[r] != 0u;
            if (__ballot(any1) == 0ull) {
#pragma unroll
                for (int r = 0; r < R; r++) k.k2[r] = 0u;
            }
        }
        lane_best<R, RAVE>(k, lane, bk, bpos);
    }
    const uint32_t uvl = a.vl > 0 ? (uint32_t)a.vl : 0u;
    // The parallel paths merge the children's entries of both scans by key.  The reference runs its second scan
    // only at a visit whose first scan found a child, and that holds for every visit of the node when it holds for
    // the first, as long as the value sums are finite (a first-scan score is then real at every visit).  A child
    // without visits whose value sum is NOT finite scores 0 + exploration at its first visit and -inf or NaN from
    // then on, while its RAVE blend, which ignores the value sum of an unvisited node, stays real: the first scan
    // can run dry in the middle of the node's visitors.  Such a node is settled one visitor after the other
    // (wave_pick applies the rule at every visit).
    bool odd = false;
    if (RAVE) {
        bool o = false;
#pragma unroll
        for (int r = 0; r < R; r++) o |= k.part[r] && !(fabsf(k.w[r]) <= 3.0e38f);
        odd = __ballot(o) != 0ull;
    }

    bool settled = false;
    int st_replay = 0;
    // where the partition finds (child, visit number) of every visitor: all visitors chose
    // run_child, or the winner order is still in LDS buffer lds_cur, or (both -1) it is in the
    // sc_child / sc_occ arrays in device memory
    int run_child = -1, lds_cur = -1;
    bool as_slice = item.pad[0] == 1;
    const bool as_scatter = item.pad[0] == 2;
    // one boundary of this node, to be worked out ahead of time (prefetch_boundaries): into the table, nothing else
    const bool just_boundary = item.pad[0] == 4;
    int hid = as_slice || as_scatter || just_boundary ? item.pad[1] : -1, slice = item.pad[2] & 0xFFFF,
        n_slices = (item.pad[2] >> 16) & 0x3FFF;
    if (as_scatter) {
        // a part of the partition of a heavy node: the visits per child are in its context
        const int *ctx = a.hctx + (size_t)hid * kHeavyCtxInts;
#pragma unroll
        for (int r = 0; r < R; r++) cnt[r] = ctx[16 + r * kWave + lane];
        settled = true;
    }
    bool contested = false;
    int best0 = -1;
    uint32_t lk0 = 0u, lp0 = 0xFFFFFFFFu;
    if (preload == 2) {
        // the walk has made the one-winner test on these very children, and it failed
        contested = __builtin_amdgcn_readfirstlane(g_chain.e_contested) != 0;
        best0 = __builtin_amdgcn_readfirstlane(g_chain.e_best0);
        lk0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)g_chain.e_lk0);
        lp0 = (uint32_t)(__builtin_amdgcn_readfirstlane(g_chain.e_second) ? R * kWave + best0 : best0);
    } else if (!as_slice && !just_boundary && !settled && m >= kRunMin && a.vl > 0 && !odd)
        settled = single_run<R, RAVE>(a, c, lane, k, bk, bpos, soff, m, m >= kRunShareMin, cnt, run_child, contested, best0,
                                      lk0, lp0);
    if (!settled && contested && m >= kSparseMin && m < kHeavyMin && !odd) {
        settled = sparse_merge<R, RAVE>(a, c, lane, k, best0, lk0, lp0, m, lds, pl.order, cnt, pending);
        if (settled) {
            lds_cur = 0;
            if (a.stats && lane == 0) atomicAdd(a.stats + 7, 1);
        } else {
#pragma unroll
            for (int r = 0; r < R; r++) cnt[r] = 0;
        }
    }
    if (R * kWave <= kHeavyFanout) {
        if (!as_slice && !just_boundary && !settled && m >= kHeavyMin && m <= kWaterLevelMaxJ && a.vl > 0 && !odd) {
            // cut the node into slices: the others go to the queue, this wavefront takes the first
            const int K = (m + slice_size(m) - 1) / slice_size(m);  // at most kMaxSlices
            // (a node whose boundaries are being worked out ahead of time has its context already)
            int id = a.hctx_cap;
            if ((item.pad[0] == 3 || (item.pad[0] == 0 && depth == 0)) && item.pad[1] > 0) id = item.pad[1] - 1;
            else if (lane == 0) id = atomicAdd(a.hctx_n, 1);
            id = __builtin_amdgcn_readfirstlane(id);
            if (id < a.hctx_cap) {
                int slot0 = 0;
                if (lane == 0) slot0 = atomicAdd(a.sched_tail, K - 1);
                slot0 = __builtin_amdgcn_readfirstlane(slot0);
                if (slot0 + K - 1 <= a.q_cap) {
                    int *ctx = a.hctx + (size_t)id * kHeavyCtxInts;
                    if (lane == 0) {
                        ctx[0] = K;
                        ctx[1] = 0;
                    }
                    for (int j = lane; j < K - 1; j += kWave) {
                        Item it = item;
                        it.pad[0] = 1;
                        it.pad[1] = id;
                        it.pad[2] = (j + 1) | (K << 16) | (list_ok ? 0 : 1 << 30);
                        a.items_q[slot0 + j] = it;
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
                    for (int j = lane; j < K - 1; j += kWave)
                        __hip_atomic_store(a.q_ready + slot0 + j, a.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    as_slice = true;
                    hid = id;
                    slice = 0;
                    n_slices = K;
                    if (a.stats && lane == 0) atomicAdd(a.stats + 15, 1);
                } else if (lane == 0) {
                    atomicExch(a.sched_wait + 1, 2);  // queue overflow: cannot happen on a tree
                }
            }
        }
        if (as_slice || just_boundary) {
            int *ctx = a.hctx + (size_t)hid * kHeavyCtxInts;
            const int S = just_boundary ? item.pad[2] >> 8 : slice_size(m);
            const bool last = slice == n_slices - 1;
            int ct_hi[R], ct_lo[R];
#pragma unroll
            for (int r = 0; r < R; r++) ct_hi[r] = ct_lo[r] = 0;
            bool ok = true;
            int rank_hi = 0, rank_lo = m;
            uint32_t T_hi = 0xFFFFFFFFu, T_lo = 0u;
            const long long ts0 = a.trace ? wall_clock64() : 0ll;
            long long ts1 = ts0;
            // The boundary behind this slice, then the one before it, both through the node's boundary table
            // (slice_boundary): the neighbours use the same numbers by construction, nobody works the same
            // boundary out twice, and a boundary worked out ahead of time is simply there.  The boundary behind
            // the last slice lies at or after the node's last visitor: with it that slice knows its one batch
            // like every other (it keeps what it needs) instead of searching for it in the batch loop.
            // (One call site, run twice: the code behind it is the largest of the kernel.)
#pragma nounroll
            for (int pass = 0; pass < 2; pass++) {
                const int b = just_boundary ? (pass == 0 ? (item.pad[2] & 255) : 0) : (pass == 0 ? slice + 1 : slice);
                if (b == 0 || !ok) continue;
                int ct[R], rank = 0;
                uint32_t T = 0u;
                ok = slice_boundary<R, RAVE>(a, c, lane, k, lds, hid, b, S, ct, T, rank);
                if (pass == 0) {
#pragma unroll
                    for (int r = 0; r < R; r++) ct_lo[r] = ct[r];
                    T_lo = T;
                    rank_lo = rank;
                } else {
#pragma unroll
                    for (int r = 0; r < R; r++) ct_hi[r] = ct[r];
                    T_hi = T;
                    rank_hi = rank;
                }
            }
            if (just_boundary) return kStepParked;
            bool preset_ok = !last;
            if (ok) {
                int sum = 0;
                bool bad = false;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    sum += ct_lo[r];
                    if (ct_lo[r] < ct_hi[r]) bad = true;
                }
                rank_lo = wave_sum_i32(sum);
                const bool broken = T_lo > T_hi || __ballot(bad) != 0ull;
                if (last) {
                    // counts that do not reach the last visitor, or thresholds out of order: the batch loop
                    // finds the end of the node by itself
                    preset_ok = !broken && rank_lo >= m;
                    if (!preset_ok) rank_lo = m;
                } else if (broken) {
                    ok = false;
                }
            }
            if (a.trace) ts1 = wall_clock64();
            if (a.trace && lane == 0) {
                g_slice_note[2] = -1;
                g_slice_note[3] = 0;
            }
            if (ok && rank_hi < m) {
                const bool closing = last || rank_lo >= m;
                const int todo = (closing ? m : rank_lo) - rank_hi;
                if (a.trace && lane == 0) {
                    g_slice_note[2] = preset_ok ? rank_lo - rank_hi : -1;
                    g_slice_note[3] = todo;
                }
                if (todo > 0) {
                    {
                        int unused_cur;
                        int between[R];  // entries of every child between the two thresholds
#pragma unroll
                        for (int r = 0; r < R; r++) between[r] = ct_lo[r] - ct_hi[r];
                        ok = water_level<R, RAVE>(a, c, lane, k, soff, rank_hi, todo, ct_hi, lds, cnt, false, unused_cur,
                                                  preset_ok, between, pl.order, pending);
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < R; r++) cnt[r] = ct_hi[r];
                }
                if (ok && closing) {
#pragma unroll
                    for (int r = 0; r < R; r++) ctx[16 + r * kWave + lane] = cnt[r];
                } else if (ok) {
                    bool bad = false;
#pragma unroll
                    for (int r = 0; r < R; r++)
                        if (cnt[r] != ct_lo[r]) bad = true;
                    if (__ballot(bad) != 0ull) {
                        ok = false;
                    }
                }
            }
            if (a.trace && lane == 0) {
                g_slice_note[0] = (int)(ts1 - ts0);
                g_slice_note[1] = (int)(wall_clock64() - ts1);
            }
            // The boundary before the last slice says how many of the first (K - 1) * S visitors every child takes:
            // a child that takes a thousand of them will be cut into slices itself, and its boundaries depend on
            // its own statistics only.  They are worked out from now on, by idle wavefronts, while this node's
            // slices are still being settled (prefetch_boundaries).  The first slice sees to that: it ends
            // before the slices in the middle of the order do, and nothing waits for it.
            if (RMAX * kWave <= kHeavyFanout && ok && slice == 0 && n_slices >= 3 && depth + 1 < a.max_depth) {
                int ctb[R], rank_b = 0;
                if (boundary_read<R>(a, lane, hid, n_slices - 1, 512, ctb, rank_b) && rank_b <= m)
                    prefetch_boundaries<R, RAVE>(f, a, c, lane, k, ctb, m - rank_b, depth, ctx);
            }
            if (!ok && lane == 0) atomicExch(ctx + 1, 1);
            // join: the wavefront that finishes last goes on with the node
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
            int before = 0;
            if (lane == 0) before = atomicSub(ctx + 0, 1);
            before = __builtin_amdgcn_readfirstlane(before);
            if (before != 1) return kStepParked;
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            const int failed = __hip_atomic_load(ctx + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int r = 0; r < R; r++)
                cnt[r] = failed ? 0
                                : __hip_atomic_load(ctx + 16 + r * kWave + lane, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT);
            settled = !failed;
            if (failed) st_replay = 1;
        }
    }
    if (just_boundary) return kStepParked;  // (a fan-out class that is never cut into slices)
    // (with RAVE, where every probe of the water level scores two scans per child; without it the path's code
    // costs the kernel more than its shorter probes save)
    if constexpr (R > 1 && RAVE) {
        if (!settled && contested && m >= kWaterLevelMin && m < kHeavyMin && a.vl > 0 && !odd && !as_slice &&
            !as_scatter) {
            settled = narrow_water_level<R, RAVE>(a, c, lane, k, soff, best0, lk0, lp0, m, lds, cnt, lds_cur, pl.order,
                                                  pending);
            if (settled && a.stats && lane == 0) atomicAdd(a.stats + 12, 1);
            if (!settled) {
                lds_cur = -1;
#pragma unroll
                for (int r = 0; r < R; r++) cnt[r] = 0;
            }
        }
    }
    if (!settled && m >= kWaterLevelMin && m <= kWaterLevelMaxJ && a.vl > 0 && !odd) {
        int zero[R];
#pragma unroll
        for (int r = 0; r < R; r++) zero[r] = 0;
        settled = water_level<R, RAVE>(a, c, lane, k, soff, 0, m, zero, lds, cnt, m < kHeavyMin, lds_cur, false, zero,
                                       pl.order, pending);
        if (!settled) st_replay = 1;
    }
    if (!settled) {
        // one visitor after the other
        run_child = -1;
        lds_cur = -1;
        const bool seq_lds = m < kHeavyMin;  // few enough visitors to keep their order in LDS
        if (seq_lds) close_pending(pending);  // the previous node's partition may still read that buffer
        for (int done = 0; done < m; done++) {
            int i = wave_pick<R, RAVE>(k, lane, bk, bpos);
            if (i < 0) return kStepLeaf;  // no child takes part: uniform, and then for every visitor
            if (a.vl <= 0) {
                // no virtual loss: nothing changes between visitors, they all follow the first
                if (!seq_lds) {
                    for (int j = lane; j < m; j += kWave) {
                        a.sc_child[soff + j] = i;
                        a.sc_occ[soff + j] = j;
                    }
                }
                if (lane == (i & 63)) {
#pragma unroll
                    for (int r = 0; r < R; r++)
                        if (r == (i >> 6)) cnt[r] = m;
                }
                run_child = i;
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
                        score_round<R, RAVE>(k, r, c.ep);
                    }
                }
                lane_best<R, RAVE>(k, lane, bk, bpos);
                if (seq_lds) {
                    pl.order[done] = ((uint32_t)i << 21) | (uint32_t)occ;
                } else {
                    a.sc_child[soff + done] = i;
                    a.sc_occ[soff + done] = occ;
                }
            }
        }
        if (run_child < 0 && seq_lds) lds_cur = 0;
        wave_sync_memory();
    }
    if (a.stats && lane == 0 && !as_scatter) {
        atomicAdd(a.stats + 0, 1);
        atomicAdd(a.stats + 1, settled ? 1 : 0);
        atomicAdd(a.stats + 2, settled ? m : 0);
        atomicAdd(a.stats + 3, settled ? 0 : m);
        atomicAdd(a.stats + 4, st_replay);
    }

    // ---- partition of the visitors by chosen child ----
    // this node's visitor list is written by the previous node's partition
    close_pending(pending);
    if (!list_ok) {
        if (!wait_list(a, off, depth, lane)) return kStepParked;
        list_ok = true;
    }
    if (run_child >= 0 && !as_scatter && !as_slice && m < kHeavyMin && a.vl > 0) {
        // Every visitor follows one child: nothing to share out.  The helpers walk down from that child for as
        // long as the visitors stay together, and write the path entries of all those levels, this node's
        // included (chain_walk, chain_finish); the owner takes the walk's barriers with them (owner_loop).
        int tn = 0;
#pragma unroll
        for (int r = 0; r < R; r++)
            if (r == (run_child >> 6)) tn = k.n[r];
        const int np_next = __builtin_amdgcn_readlane(tn, run_child & 63);
        const int child = c.cb + run_child;
        const int2 child_span = f.span[child];
        if (lane == 0) {
            TeamCmd &cm = lds.cmd;
            cm.op = kOpChain;
            cm.c_node = child;
            cm.c_np = np_next;
            cm.c_cb = child_span.x;
            cm.c_cc = child_span.y;
            cm.c_depth = depth + 1;
            cm.c_off = off;
            cm.c_m = m;
            g_chain.nodes[0] = child;
            g_chain.n_barriers = -1;
            atomicAdd(f.VL + child, (int)((uint32_t)a.vl * (uint32_t)m));
        }
        __syncthreads();  // the request is open; the owner takes part in its barriers
        next.node = child;
        next.off = off;
        next.m = m;
        next.np = np_next;
        next.span = child_span;
        next.ahead = false;
        next.chain_open = true;
        return kStepDescended;
    }
    // (1) from the visits per child: the segment of every child, in LDS for all lanes
    uint32_t lmax = 0u;
#pragma unroll
    for (int r = 0; r < R; r++) lmax = umax32(lmax, (uint32_t)cnt[r]);
    const uint32_t gmax = wave_max_u32(lmax);
    uint32_t lidx = 0xFFFFFFFFu;
#pragma unroll
    for (int r = R - 1; r >= 0; r--)
        if ((uint32_t)cnt[r] == gmax) lidx = (uint32_t)(r * kWave + lane);
    // This wavefront walks on with the largest part; the other parts go to the work queue,
    // where idle wavefronts pick them up at once.
    const int keep = gmax >= 2u ? (int)wave_min_u32(lidx) : -1;
    // where the walk goes on: ask for that node's child range now, it arrives during the scatter
    int2 keep_span = int2{0, 0};
    if (keep >= 0) keep_span = f.span[c.cb + keep];
    // A node of ordinary size whose winner order is at hand: a helper wavefront of the block
    // shares out the visitors and publishes the other children (partition_async), this one
    // walks on into the kept child at once.  What the kept child needs of that work, its
    // visitor list, it needs last (close_pending).
    if (!as_scatter && !as_slice && ((m < kHeavyMin && lds_cur >= 0) || (run_child >= 0 && m < kRunShareMin))) {
        int carry = 0, ex_keep = 0, np_keep = 0;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int inc = wave_inclusive_sum(cnt[r], lane);
            const int ex = carry + inc - cnt[r];
            const int i = r * kWave + lane;
            pl.offs[i] = ex;
            pl.cnt[i] = cnt[r];
            pl.np[i] = k.n[r];
            if (i == keep) {
                ex_keep = ex;
                np_keep = k.n[r];
            }
            carry += __builtin_amdgcn_readlane(inc, 63);
        }
        const int np_next = keep >= 0 ? __builtin_amdgcn_readlane(np_keep, keep & 63) : 0;
        const int off_next = keep >= 0 ? off + __builtin_amdgcn_readlane(ex_keep, keep & 63) : 0;
        const bool ahead_next = RMAX > 1 && keep >= 0 && depth + 1 < a.max_depth;
        if (lane == 0) {
            TeamCmd &cm = lds.cmd;
            cm.op = kOpPartition;
            cm.rounds = R;
            cm.j_cb = c.cb;
            cm.j_off = off;
            cm.j_m = m;
            cm.j_depth = depth;
            cm.j_keep = keep;
            cm.j_run_child = run_child;
            cm.pre_node = ahead_next ? c.cb + keep : -1;
            cm.pre_np = np_next;
            cm.pre_cc = -1;
        }
        __syncthreads();  // the request is open until close_pending
        pending = true;
        next.node = -1;
        next.ahead = false;
        next.chain_open = false;
        if (keep >= 0) {
            next.node = c.cb + keep;
            next.off = off_next;
            next.m = (int)gmax;
            next.np = np_next;
            next.span = keep_span;
            next.ahead = ahead_next;
        }
        return kStepDescended;
    }

    // the queue slots this node needs, asked for with one atomic per queue: a slot in the
    // single-visitor queue for every child with one visitor (in child order), a slot in the
    // work queue for every other child with visitors that this wavefront does not keep
    int n_lone = 0, n_push = 0;
    uint64_t has[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i = r * kWave + lane;
        const uint64_t lm1 = __ballot(cnt[r] == 1);
        lds.st_vl[i] = n_lone + __popcll(lm1 & ((1ull << lane) - 1ull));
        n_lone += __popcll(lm1);
        has[r] = __ballot(cnt[r] > 1 && i != keep);
        n_push += __popcll(has[r]);
    }
    int lone0 = 0, slot0 = -1;
    bool have_slots = false;
    if (!as_scatter && (m < kHeavyMin || R * kWave > kHeavyFanout)) {
        // not a node whose scatter is shared out: the answers arrive during the next steps
        if (lane == 0) {
            if (n_lone > 0) lone0 = atomicAdd(a.n_singles, n_lone);
            if (n_push > 0) slot0 = atomicAdd(a.sched_tail, n_push);
        }
        have_slots = true;
    }
    int carry = 0;
    int keep_np = 0;
    int excl[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        int inc = wave_inclusive_sum(cnt[r], lane);
        excl[r] = carry + inc - cnt[r];
        int i = r * kWave + lane;
        lds.offs[i] = excl[r];
        lds.st_j0[i] = cnt[r];
        lds.st_n[i] = k.n[r];
        if (i == keep) keep_np = k.n[r];
        carry += __builtin_amdgcn_readlane(inc, 63);
    }
    wave_sync_memory();

    // (2) the scatter; for a heavy node it is shared out in parts of the visitor list, again
    // through the queue, and the wavefront that finishes last goes on
    int r0 = 0, r1 = m;
    bool shared = false;
    if (R * kWave <= kHeavyFanout) {
        int part = 0, n_parts = 1;
        if (as_scatter) {
            part = slice;
            n_parts = n_slices;
            shared = true;
            lone0 = a.hctx[(size_t)hid * kHeavyCtxInts + 3];
            have_slots = true;  // the wavefront that finishes the scatter asks for the work queue's
        } else if (m >= kHeavyMin) {
            if (hid < 0) {
                int id = a.hctx_cap;
                if (lane == 0) id = atomicAdd(a.hctx_n, 1);
                id = __builtin_amdgcn_readfirstlane(id);
                if (id < a.hctx_cap) hid = id;
            }
            const int K2 = (m + kScatterPart - 1) / kScatterPart < kWave ? (m + kScatterPart - 1) / kScatterPart : kWave;
            // The children with several visitors are published together with the parts, before
            // their lists exist (kind 3: they wait for list_flag where they need the list; the
            // parts sit before them in the queue, so whatever a waiting child depends on has
            // been taken by a wavefront that does not wait).  None is kept: the wavefront that
            // finishes the scatter is any of those that took a part.
            uint64_t kids[R];
            int n_kids = 0;
#pragma unroll
            for (int r = 0; r < R; r++) {
                kids[r] = __ballot(cnt[r] > 1);
                n_kids += __popcll(kids[r]);
            }
            if (hid >= 0) {
                int slot0 = 0;
                if (lane == 0) slot0 = atomicAdd(a.sched_tail, K2 - 1 + n_kids);
                slot0 = __builtin_amdgcn_readfirstlane(slot0);
                if (slot0 + K2 - 1 + n_kids <= a.q_cap) {
                    int *ctx = a.hctx + (size_t)hid * kHeavyCtxInts;
#pragma unroll
                    for (int r = 0; r < R; r++) ctx[16 + r * kWave + lane] = cnt[r];
                    if (lane == 0 && n_lone > 0) lone0 = atomicAdd(a.n_singles, n_lone);
                    lone0 = __builtin_amdgcn_readfirstlane(lone0);
                    have_slots = true;
                    if (lane == 0) {
                        ctx[2] = K2;
                        ctx[3] = lone0;
                    }
                    if (lane < K2 - 1) {
                        Item it = item;
                        it.pad[0] = 2;
                        it.pad[1] = hid;
                        it.pad[2] = (lane + 1) | (K2 << 16);
                        a.items_q[slot0 + lane] = it;
                    }
                    int kslot[R];
                    int kbase = slot0 + K2 - 1;
                    // children whose boundaries are being worked out ahead of time have a context already
                    const bool ahead_ctx =
                        __hip_atomic_load(ctx + 5, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == a.epoch;
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const int i = r * kWave + lane;
                        kslot[r] = -1;
                        if (cnt[r] > 1) {
                            Item it;
                            it.node = c.cb + i;
                            it.off = off + excl[r];
                            it.m = cnt[r];
                            it.np = k.n[r];
                            it.depth = depth + 1;
                            it.pad[0] = 3;
                            it.pad[1] = ahead_ctx ? __hip_atomic_load(ctx + 16 + kHeavyFanout + i, __ATOMIC_RELAXED,
                                                                      __HIP_MEMORY_SCOPE_AGENT)
                                                  : 0;
                            it.pad[2] = 0;
                            kslot[r] = kbase + __popcll(kids[r] & ((1ull << lane) - 1ull));
                            a.items_q[kslot[r]] = it;
                        }
                        kbase += __popcll(kids[r]);
                        if (cnt[r] > 0 && a.vl > 0)
                            atomicAdd(f.VL + c.cb + i, (int)((uint32_t)a.vl * (uint32_t)cnt[r]));
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
                    if (lane < K2 - 1)
                        __hip_atomic_store(a.q_ready + slot0 + lane, a.epoch, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int r = 0; r < R; r++)
                        if (kslot[r] >= 0)
                            __hip_atomic_store(a.q_ready + kslot[r], a.epoch, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT);
                    n_parts = K2;
                    shared = true;
                } else if (lane == 0) {
                    atomicExch(a.sched_wait + 1, 2);  // queue overflow: cannot happen on a tree
                }
            }
        }
        if (shared) {
            const int per = (((m + n_parts - 1) / n_parts) + kWave - 1) & ~(kWave - 1);
            r0 = part * per < m ? part * per : m;
            r1 = r0 + per < m ? r0 + per : m;
        }
    }
    if (!have_slots && lane == 0) {  // a heavy node that could not share its scatter
        if (n_lone > 0) lone0 = atomicAdd(a.n_singles, n_lone);
        if (n_push > 0) slot0 = atomicAdd(a.sched_tail, n_push);
    }
    lone0 = __builtin_amdgcn_readfirstlane(lone0);
    int *path_next = a.paths + (size_t)(depth + 1) * a.stride;
    // kScatterUnroll chunks of 64 visitors at a time: their loads are issued together, so the
    // loop pays the memory latency once per group of chunks instead of once per chunk
    for (int base = r0; base < r1; base += kScatterUnroll * kWave) {
        int tt[kScatterUnroll], ii[kScatterUnroll], oo[kScatterUnroll];
#pragma unroll
        for (int u = 0; u < kScatterUnroll; u++) {
            const int j = base + u * kWave + lane;
            const bool in = j < r1;
            tt[u] = in ? seg_in[off + j] : 0;
            if (run_child >= 0) {
                ii[u] = run_child;
                oo[u] = j;
            } else if (lds_cur >= 0) {
                const uint32_t pay = in ? pl.order[j] : 0u;
                ii[u] = (int)((pay >> 21) & 1023u);
                oo[u] = (int)(pay & 0x1FFFFFu);
            } else {
                ii[u] = in ? a.sc_child[soff + j] : 0;
                oo[u] = in ? a.sc_occ[soff + j] : 0;
            }
        }
#pragma unroll
        for (int u = 0; u < kScatterUnroll; u++) {
            if (base + u * kWave >= r1) break;
            const bool in = base + u * kWave + lane < r1;
            const int t = tt[u], i = ii[u];
            if (in) {
                path_next[t] = c.cb + i;
                seg_out[off + lds.offs[i] + oo[u]] = t;
                // a visitor that is now alone goes to the single-visitor walk
                if (lds.st_j0[i] == 1) {
                    Item it;
                    it.node = c.cb + i;
                    it.off = t;
                    it.m = 1;
                    it.np = lds.st_n[i];
                    it.depth = depth + 1;
                    it.pad[0] = it.pad[1] = it.pad[2] = 0;
                    a.singles_q[lone0 + lds.st_vl[i]] = it;
                }
            }
        }
    }
    if (shared) {
        int *ctx = a.hctx + (size_t)hid * kHeavyCtxInts;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        int before = 0;
        if (lane == 0) before = atomicSub(ctx + 2, 1);
        before = __builtin_amdgcn_readfirstlane(before);
        if (before != 1) return kStepParked;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        // every part is written, and the children are in the queue already: tell them that
        // their lists are complete
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
#pragma unroll
        for (int r = 0; r < R; r++)
            if (cnt[r] > 1)
                __hip_atomic_store(a.list_flag + off + excl[r], depth + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // ... and the walkers of the persistent launch that their lone visitors are there
#pragma unroll
        for (int r = 0; r < R; r++)
            if (cnt[r] == 1)
                __hip_atomic_store(a.single_ready + lone0 + lds.st_vl[r * kWave + lane], a.epoch, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        if (n_lone > 0 && lane == 0) atomicSub(a.sched_wait, n_lone);
        next.node = -1;
        wave_sync_memory();
        return kStepDescended;
    }

    // (3) virtual loss of the chosen children, and the parts with several visitors that this
    // wavefront does not keep become items of the queue: everything they refer to is written,
    // make it visible to the whole device, then mark them ready
    int myslot[R];
    const int n_pushed = n_push;
    if (n_push > 0) {
        slot0 = __builtin_amdgcn_readfirstlane(slot0);
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i = r * kWave + lane;
        myslot[r] = -1;
        if (cnt[r] > 1 && i != keep) {
            int slot = slot0 + __popcll(has[r] & ((1ull << lane) - 1ull));
            if (slot < a.q_cap) {
                Item it;
                it.node = c.cb + i;
                it.off = off + excl[r];
                it.m = cnt[r];
                it.np = k.n[r];
                it.depth = depth + 1;
                it.pad[0] = it.pad[1] = it.pad[2] = 0;
                a.items_q[slot] = it;
                myslot[r] = slot;
            } else {
                atomicExch(a.sched_wait + 1, 2);  // queue overflow: cannot happen on a tree
            }
        }
        slot0 += __popcll(has[r]);
        if (cnt[r] > 0 && a.vl > 0) atomicAdd(f.VL + c.cb + i, (int)((uint32_t)a.vl * (uint32_t)cnt[r]));
    }
    if (n_pushed > 0 || n_lone > 0) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (myslot[r] >= 0)
                __hip_atomic_store(a.q_ready + myslot[r], a.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (cnt[r] == 1)
                __hip_atomic_store(a.single_ready + lone0 + lds.st_vl[r * kWave + lane], a.epoch, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (n_lone > 0 && lane == 0) atomicSub(a.sched_wait, n_lone);  // lone visitors leave the multi-visitor items
    next.node = -1;
    if (keep >= 0) {
        next.node = c.cb + keep;
        next.off = off + lds.offs[keep];
        next.m = (int)gmax;
        next.np = __builtin_amdgcn_readlane(keep_np, keep & 63);
        next.span = keep_span;
    }
    // the next step of the walk reads seg_out and reuses the LDS scratch
    wave_sync_memory();
    return kStepDescended;
}

// Multi-visitor items: a persistent kernel over a device-side work queue.  A wavefront takes
// a ticket, waits until the item with that number is published (or until no visitor is
// left in any multi-visitor item), processes the node, keeps the largest part of the group
// and publishes the other parts.  Items depend only on their ancestors, so there is no
// level barrier: the critical path is the longest chain of crowded nodes.  Every wait is
// bounded: a wavefront that polls spin_limit times raises the abort flag and all leave.
//
// A block is a team: its first wavefront (the owner) runs this loop, the other wavefronts
// wait at a block barrier until the owner shares out the batch work of a node (team_help).
template <int RMAX, bool RAVE>
__device__ __forceinline__ void owner_loop(const ForestDev &f, const SelectArgs &a, WaveLds<RMAX> &s_lds,
                                           PartLds<RMAX> &s_part, bool &pending, int lane) {
    for (;;) {
        int ticket = 0;
        if (lane == 0) ticket = atomicAdd(a.sched_head, 1);
        ticket = __builtin_amdgcn_readfirstlane(ticket);
        if (ticket >= a.q_cap) return;
        bool got = false;
        for (int spins = 0;; spins++) {
            int rdy = 0, open = 1, ab = 0;
            if (lane == 0) {
                rdy = __hip_atomic_load(a.q_ready + ticket, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == a.epoch;
                if (!rdy && (spins & 3) == 3) {
                    open = __hip_atomic_load(a.sched_wait, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    ab = __hip_atomic_load(a.sched_wait + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            rdy = __builtin_amdgcn_readfirstlane(rdy);
            open = __builtin_amdgcn_readfirstlane(open);
            ab = __builtin_amdgcn_readfirstlane(ab);
            if (rdy) {
                got = true;
                break;
            }
            if (open <= 0 || ab) break;
            if (spins >= a.spin_limit) {
                if (lane == 0 && atomicCAS(a.sched_wait + 1, 0, 1) == 0) {
                    a.sched_wait[2] = ticket;  // which item never came, for the error message
                    a.sched_wait[3] = *a.sched_tail;
                    a.sched_wait[4] = open;
                }
                break;
            }
            for (int z = 0; z < a.poll_sleep; z++) __builtin_amdgcn_s_sleep(32);
        }
        if (!got) return;
        // polling is relaxed (an acquire per poll would drop cached lines for the whole
        // compute unit every time); one acquire once the item is there
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        Item it = a.items_q[ticket];
        if (it.depth == 0 && (it.pad[0] == 0 || it.pad[0] == 4)) {  // (items the host wrote: a root, a boundary of one)
            it.np = f.N[it.node];  // (the paths' first entries, the roots, are written when the roots are set)
        }
        bool have_span = false, chain_open = false;
        int preload = 0;  // what select_group finds of the node's children (its argument of that name)
        int2 pre_span = int2{0, 0};
        for (;;) {
            const int depth = it.depth;
            const int32_t *seg_in = depth == 0 ? a.seg0 : a.seg[(depth - 1) & 1];
            int32_t *seg_out = a.seg[depth & 1];
            const long long tr0 = a.trace ? wall_clock64() : 0ll;  // the timeline, when it is switched on
            NodeCtx c = node_ctx(f, a, it.node, it.np, have_span, pre_span);
            if (chain_open) {
                // The node settled before sent all its visitors here, and the helpers walk down from this node for
                // as long as the visitors stay together (chain_walk, chain_finish).  Their block barriers count
                // this wavefront too: it takes them, one per level and the one that ends the request, and goes
                // on where the walk stopped.
                chain_open = false;
                for (int taken = 1;; taken++) {
                    __syncthreads();
                    int nb = -1;
                    if (lane == 0) nb = __hip_atomic_load(&g_chain.n_barriers, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    nb = __builtin_amdgcn_readfirstlane(nb);
                    if (nb >= 0 && taken == nb + 1) break;
                }
                pending = true;  // the helpers are writing the path entries: the barrier that ends the request is open
                it.node = __builtin_amdgcn_readfirstlane(g_chain.e_node);
                it.np = __builtin_amdgcn_readfirstlane(g_chain.e_np);
                it.depth = __builtin_amdgcn_readfirstlane(g_chain.e_depth);
                have_span = true;
                pre_span = int2{__builtin_amdgcn_readfirstlane(g_chain.e_cb), __builtin_amdgcn_readfirstlane(g_chain.e_cc)};
                preload = __builtin_amdgcn_readfirstlane(g_chain.e_kids) ? 2 : 0;
                continue;
            }
            const int preload_now = preload;
            preload = 0;
            // a boundary to work out ahead of time, of a node that turns out to have no children to choose from
            if (it.pad[0] == 4 && !(c.cc > 0 && depth < a.max_depth)) break;
            int status = kStepLeaf;
            Continuation next;
            next.node = -1;
            next.ahead = false;
            next.chain_open = false;
            if (c.cc > 0 && depth < a.max_depth) {
                if (c.cc <= kWave)
                    status = select_group<1, RAVE, RMAX>(f, a, c, lane, it, seg_in, seg_out,
                                                         reinterpret_cast<WaveLds<1> &>(s_lds), s_part, pending,
                                                         next, preload_now == 2 ? 2 : 0);
                else
                    status = select_group<RMAX, RAVE, RMAX>(f, a, c, lane, it, seg_in, seg_out, s_lds, s_part, pending,
                                                            next, preload_now);
            }
            if (a.trace && lane == 0) {
                const int ti = atomicAdd(a.trace_n, 1);
                if (ti < a.trace_cap) {
                    a.trace[12 * ti + 0] = tr0;
                    a.trace[12 * ti + 1] = wall_clock64();
                    a.trace[12 * ti + 2] = (long long)it.m | ((long long)depth << 32) | ((long long)it.pad[0] << 60);
                    // a slice or a part of a heavy node: its number and their number in the upper half
                    a.trace[12 * ti + 3] = (long long)it.node | ((long long)(uint32_t)it.pad[2] << 32);
                    for (int q = 0; q < 8; q++) a.trace[12 * ti + 4 + q] = 0;
                    if (it.pad[0] == 1 || it.m >= kHeavyMin) {
                        a.trace[12 * ti + 4] = (long long)(uint32_t)g_slice_note[0] | ((long long)(uint32_t)g_slice_note[1] << 32);
                        a.trace[12 * ti + 5] = (long long)(uint32_t)g_slice_note[2] | ((long long)(uint32_t)g_slice_note[3] << 32);
                    }
                }
            }
            if (status == kStepParked) break;  // a slice of a heavy node: another wavefront goes on with it
            if (status == kStepLeaf) {
                close_pending(pending);  // the visitor list comes from the previous node's partition
                if (it.pad[0] == 3 && !wait_list(a, it.off, depth, lane)) break;
                for (int j = lane; j < it.m; j += kWave) {
                    int t = seg_in[it.off + j];
                    a.leaf[t] = it.node;
                    a.path_len[t] = depth + 1;
                }
                if (lane == 0) {
                    if (c.cc > 0 && depth >= a.max_depth) atomicAdd(a.truncated, it.m);
                    atomicSub(a.sched_wait, it.m);  // these visitors are done
                }
                break;
            }
            if (next.node < 0) break;
            it.node = next.node;
            it.off = next.off;
            it.m = next.m;
            it.np = next.np;
            it.depth = depth + 1;
            it.pad[0] = it.pad[1] = it.pad[2] = 0;
            have_span = true;
            pre_span = next.span;
            preload = next.ahead ? 1 : 0;
            chain_open = next.chain_open;
        }
    }
}

// The partition of a settled node of ordinary size, by one helper wavefront, from what the
// owner left in LDS (the request, PartLds): next path entry and place in the chosen child's
// segment for every visitor, lone visitors to the single-visitor queue, virtual loss of the
// chosen children, and the children with several visitors that the owner does not keep
// become items of the work queue.
template <int R, int RMAX>
__device__ __forceinline__ void partition_async(const ForestDev &f, const SelectArgs &a, const TeamCmd &cm,
                                                PartLds<RMAX> &pl, int lane) {
    const int cb = __builtin_amdgcn_readfirstlane(cm.j_cb), off = __builtin_amdgcn_readfirstlane(cm.j_off);
    const int m = __builtin_amdgcn_readfirstlane(cm.j_m), depth = __builtin_amdgcn_readfirstlane(cm.j_depth);
    const int keep = __builtin_amdgcn_readfirstlane(cm.j_keep);
    const int run_child = __builtin_amdgcn_readfirstlane(cm.j_run_child);
    int cnt[R];
    uint64_t has[R];
    int n_lone = 0, n_push = 0;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i = r * kWave + lane;
        cnt[r] = pl.cnt[i];
        const uint64_t lm1 = __ballot(cnt[r] == 1);
        pl.lone[i] = n_lone + __popcll(lm1 & ((1ull << lane) - 1ull));
        n_lone += __popcll(lm1);
        has[r] = __ballot(cnt[r] > 1 && i != keep);
        n_push += __popcll(has[r]);
    }
    int lone0 = 0, slot0 = 0;
    if (lane == 0) {
        if (n_lone > 0) lone0 = atomicAdd(a.n_singles, n_lone);
        if (n_push > 0) slot0 = atomicAdd(a.sched_tail, n_push);
    }
    wave_sync_memory();
    lone0 = __builtin_amdgcn_readfirstlane(lone0);
    const int32_t *seg_in = depth == 0 ? a.seg0 : a.seg[(depth - 1) & 1];
    int32_t *seg_out = a.seg[depth & 1];
    int *path_next = a.paths + (size_t)(depth + 1) * a.stride;
    for (int base = 0; base < m; base += kScatterUnroll * kWave) {
        int tt[kScatterUnroll];
        uint32_t pay[kScatterUnroll];
#pragma unroll
        for (int u = 0; u < kScatterUnroll; u++) {
            const int j = base + u * kWave + lane;
            const bool in = j < m;
            tt[u] = in ? seg_in[off + j] : 0;
            pay[u] = run_child >= 0 ? ((uint32_t)run_child << 21) | (uint32_t)j : (in ? pl.order[j] : 0u);
        }
#pragma unroll
        for (int u = 0; u < kScatterUnroll; u++) {
            if (base + u * kWave + lane < m) {
                const int t = tt[u], i = (int)((pay[u] >> 21) & 1023u), occ = (int)(pay[u] & 0x1FFFFFu);
                path_next[t] = cb + i;
                seg_out[off + pl.offs[i] + occ] = t;
                if (pl.cnt[i] == 1) {
                    Item it;
                    it.node = cb + i;
                    it.off = t;
                    it.m = 1;
                    it.np = pl.np[i];
                    it.depth = depth + 1;
                    it.pad[0] = it.pad[1] = it.pad[2] = 0;
                    a.singles_q[lone0 + pl.lone[i]] = it;
                }
            }
        }
    }
    slot0 = __builtin_amdgcn_readfirstlane(slot0);
    int myslot[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i = r * kWave + lane;
        myslot[r] = -1;
        if (cnt[r] > 1 && i != keep) {
            const int slot = slot0 + __popcll(has[r] & ((1ull << lane) - 1ull));
            if (slot < a.q_cap) {
                Item it;
                it.node = cb + i;
                it.off = off + pl.offs[i];
                it.m = cnt[r];
                it.np = pl.np[i];
                it.depth = depth + 1;
                it.pad[0] = it.pad[1] = it.pad[2] = 0;
                a.items_q[slot] = it;
                myslot[r] = slot;
            } else {
                atomicExch(a.sched_wait + 1, 2);  // queue overflow: cannot happen on a tree
            }
        }
        slot0 += __popcll(has[r]);
        if (cnt[r] > 0 && a.vl > 0) atomicAdd(f.VL + cb + i, (int)((uint32_t)a.vl * (uint32_t)cnt[r]));
    }
    if (n_push > 0 || n_lone > 0) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (myslot[r] >= 0)
                __hip_atomic_store(a.q_ready + myslot[r], a.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (cnt[r] == 1)
                __hip_atomic_store(a.single_ready + lone0 + pl.lone[r * kWave + lane], a.epoch, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (n_lone > 0 && lane == 0) atomicSub(a.sched_wait, n_lone);  // lone visitors leave the multi-visitor items
}

// What a helper wavefront does with one request of its owner.
template <int R, bool RAVE, int RMAX>
__device__ __forceinline__ void team_help(const ForestDev &f, const SelectArgs &a, WaveLds<R> &lds, PartLds<RMAX> &pl,
                                          int tid, int op, int total, int keep, int goff, int cur, float ep,
                                          uint32_t uvl) {
    uint32_t *order = pl.order;
    if (op == kOpPartition) {
        if ((tid >> 6) == 1) partition_async<R, RMAX>(f, a, lds.cmd, pl, tid & 63);
    } else if (op == kOpOrder) {
        batch_order<R, RAVE, kTeam>(lds, tid, total, ep, uvl);
    } else if (op == kOpEmit) {
        batch_emit<R, kTeam>(a, lds, order, tid, total, keep, goff, cur);
    } else if (op == kOpRun) {
        const TeamCmd &cm = lds.cmd;
        const int best = __builtin_amdgcn_readfirstlane(cm.best), btk = __builtin_amdgcn_readfirstlane(cm.btk);
        const int bn = __builtin_amdgcn_readfirstlane(cm.bn), bvl = __builtin_amdgcn_readfirstlane(cm.bvl);
        const float bw = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(cm.bw)));
        const float bp = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(cm.bp)));
        const float bq2 = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(cm.bq2)));
        const uint32_t hk = (uint32_t)__builtin_amdgcn_readfirstlane((int)cm.hk);
        const uint32_t hp = (uint32_t)__builtin_amdgcn_readfirstlane((int)cm.hp);
        const uint32_t sk = (uint32_t)__builtin_amdgcn_readfirstlane((int)cm.sk);
        const uint32_t spos = (uint32_t)__builtin_amdgcn_readfirstlane((int)cm.spos);
        const bool proven = __builtin_amdgcn_readfirstlane(cm.proven) != 0;
        batch_run<R, RAVE, kTeam>(a, lds, tid, total, goff, best, btk, bn, bw, bp, bvl, bq2, ep, uvl, hk, hp, sk, spos,
                                  proven);
    }
}

template <int RMAX, bool RAVE>
__device__ void walkers_loop(ForestDev f, SelectArgs a, int lane);

template <int RMAX, bool RAVE>
__global__ __launch_bounds__(kTeam) void k_select_groups(ForestDev f, SelectArgs a) {
    __shared__ WaveLds<RMAX> s_lds;
    __shared__ PartLds<RMAX> s_part;
    const int tid = threadIdx.x;
    // three time stamps of the launch (100 MHz clock, low 31 bits): when its first block started, when the
    // last team left, when the last walker left
    if (blockIdx.x == 0 && tid == 0) a.times[0] = (int)(wall_clock64() & 0x7FFFFFFF);
    if ((int)blockIdx.x >= a.n_team_blocks) {
        walkers_loop<RMAX, RAVE>(f, a, tid & 63);
        if ((tid & 63) == 0) atomicMax(a.times + 2, (int)(wall_clock64() & 0x7FFFFFFF));
        return;
    }
    if (tid < kWave) {
        // every path out of the owner's loop comes back here: the helpers are always released
        bool pending = false;
        owner_loop<RMAX, RAVE>(f, a, s_lds, s_part, pending, tid);
        close_pending(pending);
        if (tid == 0) atomicMax(a.times + 1, (int)(wall_clock64() & 0x7FFFFFFF));
        if (tid == 0) s_lds.cmd.op = kOpExit;
        __syncthreads();
        return;
    }
    for (;;) {
        __syncthreads();  // the owner has written a request
        const int op = __builtin_amdgcn_readfirstlane(s_lds.cmd.op);
        if (op == kOpExit) return;
        const int rounds = __builtin_amdgcn_readfirstlane(s_lds.cmd.rounds);
        const int total = __builtin_amdgcn_readfirstlane(s_lds.cmd.total);
        const int keep = __builtin_amdgcn_readfirstlane(s_lds.cmd.keep);
        const int goff = __builtin_amdgcn_readfirstlane(s_lds.cmd.goff);
        const int cur = __builtin_amdgcn_readfirstlane(s_lds.cmd.cur);
        const float ep = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(s_lds.cmd.ep)));
        const uint32_t uvl = (uint32_t)__builtin_amdgcn_readfirstlane((int)s_lds.cmd.uvl);
        if (op == kOpChain) {
            // the helpers walk down from the child that all visitors of the owner's node follow, for as long as
            // they stay together (three of them in lockstep on a layout with wide nodes, one alone otherwise);
            // the owner goes on at the barrier that follows the walk, the path entries are written after it
            // (the request stays open until the owner needs what they write: close_pending)
            const TeamCmd &cm = s_lds.cmd;
            const KernArgsP ka = (KernArgsP)__builtin_amdgcn_kernarg_segment_ptr();
            const int wi = (tid >> 6) - 1;
            const int c_depth = __builtin_amdgcn_readfirstlane(cm.c_depth), c_m = __builtin_amdgcn_readfirstlane(cm.c_m);
            const int c_off = __builtin_amdgcn_readfirstlane(cm.c_off);
            int levels = 0;
            if (RMAX > 1 || wi == 0)
                levels = chain_walk<RMAX, RAVE>(ka, (LdsBytesP)&s_lds, wi, tid & 63, __builtin_amdgcn_readfirstlane(cm.c_node),
                                                __builtin_amdgcn_readfirstlane(cm.c_np),
                                                __builtin_amdgcn_readfirstlane(cm.c_cb),
                                                __builtin_amdgcn_readfirstlane(cm.c_cc), c_depth, c_m);
            __syncthreads();  // the walk has stopped
            if (RMAX > 1) chain_finish(ka, tid - kWave, kChainWalkers * kWave, levels, c_depth - 1, c_off, c_m);
            else if (wi == 0) chain_finish(ka, tid & 63, kWave, levels, c_depth - 1, c_off, c_m);
            __syncthreads();  // the request is done
            continue;
        }
        if (RMAX > 1 && (op == kOpPartition || op == kOpLoad) && (tid >> 6) >= 2) {
            const int pn = __builtin_amdgcn_readfirstlane(s_lds.cmd.pre_node);
            if (pn >= 0)
                load_ahead<RMAX, RAVE>(f, a, s_lds, pn, __builtin_amdgcn_readfirstlane(s_lds.cmd.pre_np),
                                       __builtin_amdgcn_readfirstlane(s_lds.cmd.pre_cb),
                                       op == kOpLoad ? __builtin_amdgcn_readfirstlane(s_lds.cmd.pre_cc) : -1, tid >> 6,
                                       tid & 63);
        }
        if (rounds == 1)
            team_help<1, RAVE, RMAX>(f, a, reinterpret_cast<WaveLds<1> &>(s_lds), s_part, tid, op, total, keep, goff, cur,
                                     ep, uvl);
        else
            team_help<RMAX, RAVE, RMAX>(f, a, s_lds, s_part, tid, op, total, keep, goff, cur, ep, uvl);
        __syncthreads();  // the request is done
    }
}

// Single visitors: the rest of the path is private to the visitor, one wavefront walks it.
// One lone visitor from its item to its leaf.  MODE 0: plain loads; 1: AHEAD; 2: AHEAD and FAST
// (select_single).
template <int RMAX, bool RAVE, int MODE>
__device__ __forceinline__ void walk_single(const ForestDev &f, const SelectArgs &a, const Item &it, int lane) {
    constexpr bool AHEAD = MODE >= 1, FAST = MODE >= 2;
    int node = it.node;
    const int t = it.off;
    int d = it.depth;
    int np = it.np;
    if (d == 0) {
        np = f.N[node];
        if (lane == 0) a.paths[t] = node;
    }
    // the widest fan-out class has no registers to spare for the child ranges
    constexpr bool kFastWide = FAST && RMAX <= 6;
    bool have_span = false;
    int2 span = int2{0, 0};
    for (;;) {
        NodeCtx c = node_ctx(f, a, node, np, have_span, span);
        int i = -1;
        int np_child = 0;
        if (c.cc > 0 && d < a.max_depth) {
            if (c.cc <= kWave) {
                i = select_single<1, RAVE, AHEAD, FAST>(f, a, c, lane, np_child, span);
                have_span = FAST;
            } else {
                i = select_single<RMAX, RAVE, AHEAD, kFastWide>(f, a, c, lane, np_child, span);
                have_span = kFastWide;
            }
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

// The kernel of a select whose traversals are all alone at their roots (one per tree): the
// walkers are the `seeded` entries the host prepared, no other launch belongs to the select, and
// one thread leaves the scheduler words as a reset would have.
template <int RMAX, bool RAVE, int MODE>
__global__ __launch_bounds__(256) void k_select_singles(ForestDev f, SelectArgs a, int seeded) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wave == 0 && lane == 0) {
        *a.n_singles = seeded;
        *a.truncated_next = 0;
        a.sched_wait[1] = 0;
    }
    if (wave >= seeded) return;
    walk_single<RMAX, RAVE, MODE>(f, a, a.singles0[wave], lane);
}

// The same walk by a whole block, for a batch of few traversals on a wide layout (a legal mask: one slot per
// action): wavefront w of the block takes round w of every node's children (64 slots), so a level costs the
// loads and the score arithmetic of ONE round instead of RMAX, one LDS exchange and one block barrier.  A few
// hundred lone walkers leave the machine empty anyway (one wavefront each on a thousand SIMDs), and what
// a walk takes is its chain of levels: memory latency plus the instruction issue of the wavefront that scores
// the children.  Same arithmetic on the same inputs (child_keys), same choice: the first maximum over the
// first-scan candidates, then the second-scan candidates (comes_before), the second scan only with a real
// first-scan score, the least visited participating child when no candidate has a real score (wave_pick).
struct SingleSlot {
    uint32_t bk, bpos;    // the wavefront's best candidate (key 0 = none)
    int bn, bsx, bsy;     // that child's visit count and child range
    uint32_t any1;        // one of its children has a real first-scan key
    uint32_t fn, fidx;    // its least visited participating child (visit count as an ordered uint; ~0 = none)
    int fcn, fsx, fsy;    // that child's visit count and child range
};

template <int RMAX, bool RAVE>
__global__ __launch_bounds__(RMAX * kWave) void k_select_singles_team(ForestDev f, SelectArgs a, int seeded) {
    constexpr int F = RMAX * kWave;
    __shared__ SingleSlot slot[2][RMAX];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        *a.n_singles = seeded;
        *a.truncated_next = 0;
        a.sched_wait[1] = 0;
    }
    if ((int)blockIdx.x >= seeded) return;
    const Item it = a.singles0[blockIdx.x];
    int node = it.node, d = it.depth, np = it.np;
    const int t = it.off;
    if (d == 0) {
        np = f.N[node];
        if (threadIdx.x == 0) a.paths[t] = node;
    }
    int2 span = f.span[node];
    for (int level = 0;; level++) {
        const int cb = span.x, cc = span.y;
        int nelig = cc;
        if (a.pw) {
            const int kk = ceil_sqrt_i32(np);
            nelig = kk < cc ? kk : cc;
        }
        const float ep = a.c_puct * sqrtf((float)np);
        int ci = -1, np_child = 0;
        int2 span_child = int2{0, 0};
        if (cc > 0 && d < a.max_depth) {
            // this wavefront's round of the children: everything asked for at once
            const int i = wv * kWave + lane;
            const bool in = i < nelig;
            const int id = cb + i;
            uint32_t word = 0xFFFFFFFFu;
            int n = 0, vl = 0;
            float w = 0.0f, p = 0.0f, q2 = 0.0f;
            int2 sp = int2{0, 0};
            if (wv * kWave < nelig) {  // uniform
                if (in && f.legal) word = f.legal[(uint32_t)id >> 5];
                if (in) {
                    n = f.N[id];
                    w = f.W[id];
                    p = f.P[id];
                    vl = f.VL[id];
                    if (RAVE) q2 = f.q2[id];
                    sp = f.span[id];
                }
            }
            const bool part = in && ((word >> ((uint32_t)id & 31u)) & 1u);
            uint32_t k1 = 0u, k2 = 0u;
            if (part) child_keys<RAVE>(n, w, p, vl, q2, ep, k1, k2);
            uint32_t bk = k1, bpos = (uint32_t)i;
            if (k2 > bk) {
                bk = k2;
                bpos = (uint32_t)(F + i);
            }
            if (bk == 0u) bpos = 0xFFFFFFFFu;
            uint32_t hk, hp;
            wave_best(bk, bpos, hk, hp);
            const uint32_t mn = part ? (uint32_t)n ^ 0x80000000u : 0xFFFFFFFFu;
            const uint32_t gm = wave_min_u32(mn);
            const uint32_t gidx = wave_min_u32(part && mn == gm ? (uint32_t)i : 0xFFFFFFFFu);
            const bool any1 = __ballot(k1 != 0u) != 0ull;
            const int bl = hk != 0u ? (int)((hp >= (uint32_t)F ? hp - (uint32_t)F : hp) & 63u) : 0;
            const int fl = gidx != 0xFFFFFFFFu ? (int)(gidx & 63u) : 0;
            const int bn = __builtin_amdgcn_readlane(n, bl), bsx = __builtin_amdgcn_readlane(sp.x, bl);
            const int bsy = __builtin_amdgcn_readlane(sp.y, bl);
            const int fcn = __builtin_amdgcn_readlane(n, fl), fsx = __builtin_amdgcn_readlane(sp.x, fl);
            const int fsy = __builtin_amdgcn_readlane(sp.y, fl);
            if (lane == 0) {
                SingleSlot &sl = slot[level & 1][wv];
                sl.bk = hk;
                sl.bpos = hp;
                sl.bn = bn;
                sl.bsx = bsx;
                sl.bsy = bsy;
                sl.any1 = any1 ? 1u : 0u;
                sl.fn = gm;
                sl.fidx = gidx;
                sl.fcn = fcn;
                sl.fsx = fsx;
                sl.fsy = fsy;
            }
            __syncthreads();  // (the slots alternate with the level: nobody is a level ahead of a reader)
            // ---- the same over the wavefronts ----
            uint32_t gk = 0u, gp = 0xFFFFFFFFu, a1 = 0u, fn = 0xFFFFFFFFu, fi = 0xFFFFFFFFu;
            int won = 0, fwon = 0;
#pragma unroll
            for (int x = 0; x < RMAX; x++) {
                const SingleSlot &sl = slot[level & 1][x];
                a1 |= sl.any1;
                if (sl.bk != 0u && comes_before(sl.bk, sl.bpos, gk, gp)) {
                    gk = sl.bk;
                    gp = sl.bpos;
                    won = x;
                }
                if (sl.fn < fn || (sl.fn == fn && sl.fidx < fi)) {
                    fn = sl.fn;
                    fi = sl.fidx;
                    fwon = x;
                }
            }
            if (RAVE && gk != 0u && gp >= (uint32_t)F && a1 == 0u) gk = 0u;  // no second scan without a first-scan score
            if (gk != 0u) {
                const SingleSlot &sl = slot[level & 1][won];
                ci = (int)(gp >= (uint32_t)F ? gp - (uint32_t)F : gp);
                np_child = sl.bn;
                span_child = int2{sl.bsx, sl.bsy};
            } else if (fi != 0xFFFFFFFFu) {
                const SingleSlot &sl = slot[level & 1][fwon];
                ci = (int)fi;
                np_child = sl.fcn;
                span_child = int2{sl.fsx, sl.fsy};
            }
            ci = __builtin_amdgcn_readfirstlane(ci);
            np_child = __builtin_amdgcn_readfirstlane(np_child);
            span_child.x = __builtin_amdgcn_readfirstlane(span_child.x);
            span_child.y = __builtin_amdgcn_readfirstlane(span_child.y);
        }
        if (ci < 0) {
            if (threadIdx.x == 0) {
                a.leaf[t] = node;
                a.path_len[t] = d + 1;
                if (cc > 0 && d >= a.max_depth) atomicAdd(a.truncated, 1);
            }
            return;
        }
        const int child = cb + ci;
        if (threadIdx.x == 0) {
            if (a.stats) atomicAdd(a.stats + 6, 1);
            if (a.vl > 0) atomicAdd(f.VL + child, a.vl);
            a.paths[(size_t)(d + 1) * a.stride + t] = child;
        }
        node = child;
        np = np_child;
        span = span_child;
        d++;
    }
}

// The walkers of the persistent launch: wavefronts of the blocks behind the teams take the lone
// visitors one by one as the teams create them (a ticket, then the entry's ready word, set after
// the release fence of whoever wrote the entry), so that a lone visitor walks while the chain of
// crowded nodes is still being settled.  A walker leaves when no visitor is left in any
// multi-visitor item (nothing more can come) and its ticket lies beyond the entries written.
// The wait is bounded like every other.  Not inlined (the teams' code keeps its registers) and the
// arguments by value (by reference, the kernel's own copies would have to live in memory, and every
// use of them in the teams' code would become a load).
template <int RMAX, bool RAVE>
__device__ __noinline__ void walkers_loop(ForestDev f, SelectArgs a, int lane) {
    for (;;) {
        int ticket = 0;
        if (lane == 0) ticket = atomicAdd(a.singles_head, 1);
        ticket = __builtin_amdgcn_readfirstlane(ticket);
        bool got = false;
        for (int spins = 0;; spins++) {
            int rdy = 0, open = 1, ab = 0, n = 0;
            if (lane == 0) {
                rdy = ticket < a.n_trav &&
                      __hip_atomic_load(a.single_ready + ticket, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == a.epoch;
                if (!rdy && (spins & 3) == 3) {
                    open = __hip_atomic_load(a.sched_wait, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    ab = __hip_atomic_load(a.sched_wait + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (open <= 0) {
                        // every entry was counted before its writer let go of its visitors
                        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
                        n = __hip_atomic_load(a.n_singles, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if (ticket < n) open = 1;  // counted, so its ready word is on its way
                    }
                }
            }
            rdy = __builtin_amdgcn_readfirstlane(rdy);
            open = __builtin_amdgcn_readfirstlane(open);
            ab = __builtin_amdgcn_readfirstlane(ab);
            if (rdy) {
                got = true;
                break;
            }
            if (open <= 0 || ab) break;
            if (spins >= a.spin_limit) {
                if (lane == 0 && atomicCAS(a.sched_wait + 1, 0, 4) == 0) {
                    a.sched_wait[2] = ticket;  // which entry never came, for the error message
                    a.sched_wait[3] = *a.n_singles;
                    a.sched_wait[4] = open;
                }
                break;
            }
            for (int z = 0; z < a.poll_sleep; z++) __builtin_amdgcn_s_sleep(32);
        }
        if (!got) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        const Item it = a.singles_q[ticket];
        const long long tr0 = a.trace ? wall_clock64() : 0ll;
        if (a.fast_singles) walk_single<RMAX, RAVE, 2>(f, a, it, lane);
        else walk_single<RMAX, RAVE, 0>(f, a, it, lane);
        if (a.stats && lane == 0) atomicAdd(a.stats + 11, 1);
        if (a.trace && lane == 0) {  // the timeline: a lone visitor's walk, kind 6
            const int ti = atomicAdd(a.trace_n, 1);
            if (ti < a.trace_cap) {
                a.trace[12 * ti + 0] = tr0;
                a.trace[12 * ti + 1] = wall_clock64();
                a.trace[12 * ti + 2] = 1ll | ((long long)it.depth << 32) | (6ll << 60);
                a.trace[12 * ti + 3] = (long long)it.node;
                for (int q = 0; q < 8; q++) a.trace[12 * ti + 4 + q] = 0;
            }
        }
    }
}

// Scheduler state, statistics, the work queue seeded with the items of the roots, and the
// single-visitor queue seeded with the traversals that are alone at their root.
__global__ void k_select_reset(SelectArgs a, int n_items0, int n_singles0, int open0, int n_traversals, int n_hctx0) {
    const int gid = blockIdx.x * blockDim.x + threadIdx.x;
    const int step = gridDim.x * blockDim.x;
    if (gid == 0) {
        *a.truncated = 0;
        *a.truncated_next = 0;
        *a.n_singles = n_singles0;
        *a.sched_head = 0;
        *a.singles_head = 0;
        *a.sched_tail = n_items0;
        a.sched_wait[0] = open0;
        a.sched_wait[1] = 0;
        *a.hctx_n = n_hctx0;  // the contexts of heavy roots are handed out when the roots are set
        *a.trace_n = 0;
    }
    if (a.stats && gid < 16) a.stats[gid] = 0;
    if (gid < 3) a.times[gid] = 0;
    for (int i = gid; i < n_items0; i += step) {
        a.items_q[i] = a.items0[i];
        a.q_ready[i] = a.epoch;
    }
    for (int i = gid; i < n_singles0; i += step) {
        a.singles_q[i] = a.singles0[i];
        a.single_ready[i] = a.epoch;
    }
    // a traversal that the selection does not finish (the kernel gave up) has an empty path
    for (int i = gid; i < n_traversals; i += step) {
        a.path_len[i] = 0;
        a.leaf[i] = -1;
        a.list_flag[i] = 0;
    }
}

template <int RMAX, bool RAVE>
static hipError_t launch_kernels(const ForestDev &f, const SelectArgs &a0, int n_items0, int n_traversals,
                                 int n_cus, hipStream_t s) {
    // Few walkers cannot keep the memory system busy: then the variant that spends bytes to save
    // dependent trips (select_single, FAST).  The number of lone visitors is only known on the
    // device; the number of traversals bounds it.  Measured: it pays on a board layout (legal
    // mask: three trips per level become one), not on a compact one (two become one).
    const bool fast = f.legal && n_traversals <= kFastSinglesMax;
    if (n_items0 > 0) {
        // One persistent launch: teams for the multi-visitor items (no more than there can be items
        // at once: an item has at least two visitors) and, behind them, blocks of walkers for the lone
        // visitors the teams create.  ONE block per compute unit, although two or three would fit: a
        // selection takes as long as its longest chain of crowded nodes, the wavefront that works on that
        // chain issues an instruction every few cycles at best, and every other block on its compute
        // unit (waiting for work, polling) takes issue slots, cache and LDS bandwidth from it.  Measured
        // on the 4 M-node chess-like tree: 0.247 ms a selection with two blocks per unit, 0.222 with one.
        int capacity = n_cus;
        if (capacity < 2) capacity = 2;
        int walkers = n_traversals / 64;
        if (walkers > capacity / 4) walkers = capacity / 4;
        if (walkers > kMaxWalkerBlocks) walkers = kMaxWalkerBlocks;  // idle walkers poll: more of them slow the teams
        if (walkers < 4) walkers = 4;  // (a small batch ends with a handful of lone walks: enough walkers to take them at once)
        int teams = capacity - walkers;
        const int most = n_traversals / 2;
        if (teams > most) teams = most;
        if (teams < 1) teams = 1;
        SelectArgs a = a0;
        a.n_team_blocks = teams;
        a.fast_singles = fast ? 1 : 0;
        hipLaunchKernelGGL((k_select_groups<RMAX, RAVE>), dim3(teams + walkers), dim3(kTeam), 0, s, f, a);
        return hipGetLastError();
    }
    // every traversal is alone at its root: the walkers are the host's list
    const dim3 grid((n_traversals + 3) / 4), block(256);
    if (RMAX > 1 && f.legal && n_traversals * RMAX <= kTeamSinglesMaxWaves)
        hipLaunchKernelGGL((k_select_singles_team<RMAX, RAVE>), dim3(n_traversals), dim3(RMAX * kWave), 0, s, f, a0,
                           n_traversals);
    else if (!f.legal)
        hipLaunchKernelGGL((k_select_singles<RMAX, RAVE, 0>), grid, block, 0, s, f, a0, n_traversals);
    else if (fast)
        hipLaunchKernelGGL((k_select_singles<RMAX, RAVE, 2>), grid, block, 0, s, f, a0, n_traversals);
    else
        hipLaunchKernelGGL((k_select_singles<RMAX, RAVE, 1>), grid, block, 0, s, f, a0, n_traversals);
    return hipGetLastError();
}

hipError_t launch_select(const ForestDev &f, const SelectArgs &a, int n_items0, int n_singles0, int n_traversals,
                         int max_fanout, bool rave, int n_cus, int n_hctx0, hipStream_t s) {
    // Every traversal alone at its root (one per tree: leaf-parallel self-play): the single-visitor
    // kernel is the whole select and takes its walkers from the host's list; every walker writes its
    // own leaf and path length, so nothing has to be cleared first (the statistics apart).
    // Otherwise the reset launch.
    const bool alone = n_items0 == 0 && n_singles0 == n_traversals;
    if (!alone || a.stats || a.trace) {  // (the statistics and the timeline start at zero)
        int reset_blocks = (n_traversals + 255) / 256;
        hipLaunchKernelGGL(k_select_reset, dim3(reset_blocks), dim3(256), 0, s, a, n_items0, n_singles0,
                           n_traversals - n_singles0, n_traversals, n_hctx0);
    }
#define OMK_DISPATCH(RM)                                                              \
    return rave ? launch_kernels<RM, true>(f, a, n_items0, n_traversals, n_cus, s)    \
                : launch_kernels<RM, false>(f, a, n_items0, n_traversals, n_cus, s)
    if (max_fanout <= 64) { OMK_DISPATCH(1); }
    if (max_fanout <= 256) { OMK_DISPATCH(4); }
    if (max_fanout <= 384) { OMK_DISPATCH(6); }
    OMK_DISPATCH(16);
#undef OMK_DISPATCH
}

}  // namespace omk
