// Batched PUCT selection with virtual loss over the device-resident forest.
//
// What it computes is phase 1 of MCTSEngine::executeBatchedTreeSearch run by ONE thread,
// traversals in index order (reference src/mcts/mcts_engine_batch_tree_simple.cpp:73-185):
// descend while the node is expanded, MCTSNode::selectChild (src/mcts/mcts_node.cpp:90-236),
// addVirtualLoss on the selected child (src/mcts/mcts_node_virtual_loss.cpp:15-20).
//
// How: during this phase only virtual-loss counters change, and the counter of a child
// matters only to selections made at its parent.  On a tree, the traversals that reach a
// node all come through its parent.  So a work item is (node, the list of traversals that
// reached it, in traversal-index order); ONE 64-lane wavefront owns the item, loads the
// children once (coalesced, one child per lane per round), and plays the visitors one
// after another on register-resident statistics: score, DPP arg-max with lowest-index
// tie-break, bump the chosen child's virtual loss, next visitor.  That reproduces the
// serial order exactly.  The visitors are then partitioned by chosen child (stable, so
// still in traversal order) into the work items of the next level.  An item with a single
// visitor owns its whole remaining path, so the wavefront simply walks it to the leaf.
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

// Wave-wide winner: child index, or -1 when no child takes part.  When no score beats
// -infinity the reference falls back to the least-visited child, first minimum
// (mcts_node.cpp:173-181).
template <int R, bool RAVE>
__device__ __forceinline__ int wave_pick(const Kids<R, RAVE> &k, int lane, uint32_t bk, uint32_t bpos) {
    uint32_t m = wave_max_u32(bk);
    if (m != 0u) {
        uint64_t tie = __ballot(bk == m);
        uint32_t pos;
        if (__popcll(tie) == 1) {
            int wl = __builtin_amdgcn_readfirstlane(__ffsll((long long)tie) - 1);
            pos = (uint32_t)__builtin_amdgcn_readlane((int)bpos, wl);
        } else {
            pos = wave_min_u32(bk == m ? bpos : 0xFFFFFFFFu);
        }
        return (int)(pos >= (uint32_t)(R * kWave) ? pos - (uint32_t)(R * kWave) : pos);
    }
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

// All visitors of a multi-visitor item, in order.  Writes the chosen node of every visitor
// into the path, bumps virtual loss, partitions the visitors by child into seg_out and
// appends one item per visited child to the next level's queue.
template <int R, bool RAVE>
__device__ __forceinline__ bool select_group(const ForestDev &f, const SelectArgs &a, const NodeCtx &c, int lane,
                                             int off, int m, int depth, int *s_offs) {
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

    int *path_next = a.paths + (size_t)(depth + 1) * a.stride;
    for (int base = 0; base < m; base += kWave) {
        int tj_lane = (base + lane < m) ? a.seg_in[off + base + lane] : -1;
        int lim = m - base < kWave ? m - base : kWave;
        for (int jj = 0; jj < lim; jj++) {
            int i = wave_pick<R, RAVE>(k, lane, bk, bpos);
            if (i < 0) return false;  // no child takes part: uniform, and then for every visitor
            int t = __builtin_amdgcn_readlane(tj_lane, jj);
            if (lane == (i & 63)) {
                int occ = 0;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    if (r == (i >> 6)) {
                        occ = cnt[r];
                        cnt[r] = occ + 1;
                        if (a.vl > 0) k.vl[r] = (int)((uint32_t)k.vl[r] + (uint32_t)a.vl);
                        score_round<R, RAVE>(k, r, c.ep, a.rave_k);
                    }
                }
                lane_best<R, RAVE>(k, lane, bk, bpos);
                path_next[t] = c.cb + i;
                a.sc_child[off + base + jj] = i;
                a.sc_occ[off + base + jj] = occ;
            }
        }
    }

    // exclusive prefix of the visit counts in child order -> segment of every child
    int carry = 0;
#pragma unroll
    for (int r = 0; r < R; r++) {
        int inc = wave_inclusive_sum(cnt[r], lane);
        int excl = carry + inc - cnt[r];
        int i = r * kWave + lane;
        s_offs[i] = excl;
        uint64_t has = __ballot(cnt[r] > 0);
        int nnew = __popcll(has);
        if (nnew > 0) {
            int slot0 = 0;
            if (lane == 0) slot0 = atomicAdd(a.counters + depth + 1, nnew);
            slot0 = __builtin_amdgcn_readfirstlane(slot0);
            if (cnt[r] > 0) {
                int slot = slot0 + __popcll(has & ((1ull << lane) - 1ull));
                Item it;
                it.node = c.cb + i;
                it.off = off + excl;
                it.m = cnt[r];
                it.np = k.n[r];
                a.items_out[slot] = it;
                if (a.vl > 0) atomicAdd(f.VL + c.cb + i, a.vl * cnt[r]);
            }
        }
        carry += __builtin_amdgcn_readlane(inc, 63);
    }
    // make this wave's LDS and scratch writes visible to its own other lanes
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    for (int j = lane; j < m; j += kWave) {
        int t = a.seg_in[off + j];
        int i = a.sc_child[off + j];
        a.seg_out[off + s_offs[i] + a.sc_occ[off + j]] = t;
    }
    return true;
}

template <int RMAX, bool RAVE>
__global__ __launch_bounds__(256) void k_select_level(ForestDev f, SelectArgs a, int depth) {
    __shared__ int s_offs_all[4][RMAX * kWave];
    const int lane = threadIdx.x & 63;
    const int wib = threadIdx.x >> 6;
    const int wave = blockIdx.x * 4 + wib;
    if (wave >= a.counters[depth]) return;
    const Item it = a.items_in[wave];
    int node = it.node;
    int np = it.np;
    if (depth == 0) np = f.N[node];

    if (it.m > 1) {
        NodeCtx c = node_ctx(f, a, node, np);
        bool descended = false;
        if (depth == 0) {
            for (int j = lane; j < it.m; j += kWave) a.paths[a.seg_in[it.off + j]] = node;
        }
        if (c.cc > 0 && depth < a.max_depth) {
            int *s_offs = s_offs_all[wib];
            if (c.cc <= kWave) descended = select_group<1, RAVE>(f, a, c, lane, it.off, it.m, depth, s_offs);
            else descended = select_group<RMAX, RAVE>(f, a, c, lane, it.off, it.m, depth, s_offs);
        }
        if (!descended) {
            for (int j = lane; j < it.m; j += kWave) {
                int t = a.seg_in[it.off + j];
                a.leaf[t] = node;
                a.path_len[t] = depth + 1;
            }
            if (c.cc > 0 && depth >= a.max_depth && lane == 0) atomicAdd(a.truncated, it.m);
        }
        return;
    }

    // single visitor: walk the private remainder of the path
    const int t = a.seg_in[it.off];
    int d = depth;
    if (depth == 0 && lane == 0) a.paths[t] = node;
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
            if (a.vl > 0) atomicAdd(f.VL + child, a.vl);
            a.paths[(size_t)(d + 1) * a.stride + t] = child;
        }
        node = child;
        np = np_child;
        d++;
    }
}

__global__ void k_select_reset(int *counters, int n_counters, int n_items0, int *truncated) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_counters) counters[i] = (i == 0) ? n_items0 : 0;
    if (i == 0) *truncated = 0;
}

template <int RMAX, bool RAVE>
static hipError_t launch_levels(const ForestDev &f, SelectArgs a, const BatchBuffers &b, hipStream_t s) {
    const int n_waves = b.n_traversals;
    const int grid = (n_waves + 3) / 4;
    for (int depth = 0; depth <= a.max_depth; depth++) {
        if (depth == 0) {
            a.items_in = b.items0;
            a.seg_in = b.seg0;
        } else {
            a.items_in = b.items[(depth - 1) & 1];
            a.seg_in = b.seg[(depth - 1) & 1];
        }
        a.items_out = b.items[depth & 1];
        a.seg_out = b.seg[depth & 1];
        hipLaunchKernelGGL((k_select_level<RMAX, RAVE>), dim3(grid), dim3(256), 0, s, f, a, depth);
    }
    return hipGetLastError();
}

hipError_t launch_select(const ForestDev &f, SelectArgs a, const BatchBuffers &b, int max_fanout, bool rave,
                         hipStream_t s) {
    hipLaunchKernelGGL(k_select_reset, dim3((a.max_depth + 2 + 63) / 64), dim3(64), 0, s, a.counters,
                       a.max_depth + 2, b.n_items0, a.truncated);
#define OMK_DISPATCH(RM)                                                 \
    return rave ? launch_levels<RM, true>(f, a, b, s) : launch_levels<RM, false>(f, a, b, s)
    if (max_fanout <= 64) { OMK_DISPATCH(1); }
    if (max_fanout <= 256) { OMK_DISPATCH(4); }
    if (max_fanout <= 384) { OMK_DISPATCH(6); }
    OMK_DISPATCH(16);
#undef OMK_DISPATCH
}

}  // namespace omk
