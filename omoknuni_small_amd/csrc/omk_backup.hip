// Virtual-loss apply / revert, value backup, leaf gather export and the transposition
// table probes: the scattered read-modify-write side of the search step.
//
// Node operations restated from the reference (src/mcts/mcts_node_virtual_loss.cpp):
//   addVirtualLoss(a)     :15-20   if a > 0: VL += a
//   removeVirtualLoss(a)  :32-42   if a > 0: old = VL; VL -= a; if old < a: VL = 0
//   update(v)             :54-71   N += 1; W += v; if VL > 0: VL -= 1
// and the backup loop src/mcts/mcts_engine_batch_tree_simple.cpp:276-281
//   for node in reversed(path): update(v); removeVirtualLoss(a); v = -v
//
// Counter algebra used below.  One backup visit maps VL = x to
//   a > 0 :  max(0, x - (a+1))      (x <= 0 gives 0 as well)
//   a <= 0:  x > 0 ? x - 1 : x
// and one revert maps x to max(0, x - a).  Each is a "subtract, clamp at zero" map, so m
// visits in ANY order give max(0, x - k*m): the result of the serial reference does not
// depend on the order, and "atomic subtract, then atomic max with 0 if the old value was
// too small" reaches it without a lock (after the first clamp fires the value never
// rises above 0 again, and the last operation on the address is always a clamp or a
// subtract that stayed non-negative).
#include <algorithm>

#include "omk_internal.h"

namespace omk {

__device__ __forceinline__ void vl_sub_clamp(int32_t *addr, int k) {
    int old = atomicSub(addr, k);
    if (old < k) atomicMax(addr, 0);
}

// x > 0 ? max(0, x - k) : x   (update() without a following revert)
__device__ __forceinline__ void vl_dec_if_positive(int32_t *addr, int k) {
    int old = *(volatile int32_t *)addr;
    while (old > 0) {
        int want = old > k ? old - k : 0;
        int prev = atomicCAS(addr, old, want);
        if (prev == old) break;
        old = prev;
    }
}

__global__ __launch_bounds__(256) void k_apply_vl(ForestDev f, const int32_t *paths, const int32_t *path_len, int n,
                                                  int stride, int vl) {
    int t = blockIdx.x * 256 + threadIdx.x;
    int d = blockIdx.y + 1;  // the root of a path never receives virtual loss
    if (t >= n || d >= path_len[t]) return;
    atomicAdd(f.VL + paths[(size_t)d * stride + t], vl);
}

__global__ __launch_bounds__(256) void k_revert_vl(ForestDev f, const int32_t *paths, const int32_t *path_len, int n,
                                                   int stride, int vl) {
    int t = blockIdx.x * 256 + threadIdx.x;
    int d = blockIdx.y;
    bool act = t < n && d < path_len[t];
    int node = act ? paths[(size_t)d * stride + t] : -1;
    uint64_t mask = __ballot(act);
    if (mask == 0ull) return;
    int leader = __ffsll((long long)mask) - 1;
    int node0 = __builtin_amdgcn_readlane(node, leader);
    if (__ballot(act && node != node0) == 0ull) {
        // the whole wave sits on one node (top of a single tree): one combined operation
        if ((int)(threadIdx.x & 63) == leader) vl_sub_clamp(f.VL + node0, vl * __popcll(mask));
        return;
    }
    if (act) vl_sub_clamp(f.VL + node, vl);
}

// One thread per (traversal, depth).  Many traversals of a block meet on the same nodes near
// the root (thousands of visitors on a handful of nodes), and atomics on one address are
// served one after another: the block first combines its visits per node in a small LDS
// table (count, value sum) and then issues one set of global atomics per distinct node.
constexpr int kBackupSlots = 512;  // two per thread: the table never fills

__global__ __launch_bounds__(256) void k_backup(ForestDev f, const int32_t *paths, const int32_t *path_len,
                                                const float *values, int n, int stride, int vl) {
    __shared__ int s_key[kBackupSlots];
    __shared__ int s_cnt[kBackupSlots];
    __shared__ float s_w[kBackupSlots];
    const int tid = threadIdx.x;
    int t = blockIdx.x * 256 + tid;
    int d = blockIdx.y;
    int len = t < n ? path_len[t] : 0;
    bool act = d < len;
    if (__syncthreads_or(act ? 1 : 0) == 0) return;  // nothing this deep in this block
    for (int i = tid; i < kBackupSlots; i += 256) {
        s_key[i] = -1;
        s_cnt[i] = 0;
        s_w[i] = 0.0f;
    }
    __syncthreads();
    if (act) {
        int node = paths[(size_t)d * stride + t];
        float v = values[t];
        if ((len - 1 - d) & 1) v = -v;  // the leaf receives +value, every ply up flips it
        uint32_t h = ((uint32_t)node * 2654435761u) >> 23;
        for (;;) {
            int prev = atomicCAS(&s_key[h], -1, node);
            if (prev == -1 || prev == node) break;
            h = (h + 1u) & (uint32_t)(kBackupSlots - 1);
        }
        atomicAdd(&s_cnt[h], 1);
        atomicAdd(&s_w[h], v);
    }
    __syncthreads();
    for (int i = tid; i < kBackupSlots; i += 256) {
        const int node = s_key[i];
        if (node < 0) continue;
        const int cnt = s_cnt[i];
        atomicAdd(f.N + node, cnt);
        unsafeAtomicAdd(f.W + node, s_w[i]);
        if (vl > 0) vl_sub_clamp(f.VL + node, (vl + 1) * cnt);
        else vl_dec_if_positive(f.VL + node, cnt);
    }
}

__global__ __launch_bounds__(256) void k_export(ForestDev f, const int32_t *paths, const int32_t *path_len, int n,
                                                int stride, int max_depth, int32_t *out_paths,
                                                int32_t *out_actions) {
    int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int row = max_depth + 1;
    if (g >= (int64_t)n * row) return;
    int t = (int)(g / row);
    int d = (int)(g - (int64_t)t * row);
    int len = path_len[t];
    int node = d < len ? paths[(size_t)d * stride + t] : -1;
    if (node >= f.n_nodes) node = -1;  // never index the forest with an id it does not have
    if (out_paths) out_paths[g] = node;
    if (out_actions && d >= 1) {
        int act = -1;
        if (node >= 0) act = f.action ? f.action[node] : node;
        out_actions[(int64_t)t * max_depth + d - 1] = act;
    }
}

// ---- position keys of the selected leaves: GomokuState::compute_hash_signature_internal
// (src/games/gomoku/gomoku_state.cpp:947-957) over the tables of utils::ZobristHash
// (src/utils/zobrist_hash.cpp:9-36), for the state the traversal loop rebuilds by replaying its
// move list (mcts_engine_batch_tree_simple.cpp:119-124,133-137) ----

// A stone placed stays (no captures), so the key of the replayed state is the root state's key
// with the piece keys of the path's moves folded in and the side-to-move key swapped: the mover
// of ply k is the root's side to move when k is even.  One thread per traversal; the path is
// stored level-major, so each level is a coalesced read.
__global__ __launch_bounds__(256) void k_leaf_keys(ForestDev f, const int32_t *paths, const int32_t *path_len, int n,
                                                   int stride, const uint64_t *piece, int cells,
                                                   const uint64_t *player, const uint64_t *root_key,
                                                   const int32_t *root_player, uint64_t *out, int *d_status) {
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= n) return;
    const int len = path_len[t];
    const int p0 = root_player[t] & 1;
    uint64_t h = root_key[t];
    bool bad = false;
    for (int d = 1; d < len; d++) {
        const int node = paths[(size_t)d * stride + t];
        if (node < 0 || node >= f.n_nodes) {  // never index the forest with an id it does not have
            bad = true;
            break;
        }
        const int act = f.action ? f.action[node] : node;
        if (act < 0 || act >= cells) {
            bad = true;
            break;
        }
        h ^= piece[(size_t)((p0 + d - 1) & 1) * cells + act];
    }
    if (len >= 1 && ((len - 1) & 1)) h ^= player[p0] ^ player[p0 ^ 1];
    if (len < 1) bad = true;
    out[t] = bad ? ~0ull : h;
    if (bad) atomicAdd(d_status, 1);
}

// ---- leaf expansion: MCTSNode::expand + setPriorProbabilities
// (src/mcts/mcts_node.cpp:238-436, :512-593) for a batch of leaves ----

// Bits of the legal mask for ids that did not exist before: the tail of the last old word
// and every later word up to the new end start out clear.
__global__ void k_expand_mask(uint32_t *legal, int64_t old_nodes, int64_t new_nodes) {
    const int64_t w0 = old_nodes >> 5, w1 = (new_nodes + 31) >> 5;
    for (int64_t w = w0 + blockIdx.x * (int64_t)blockDim.x + threadIdx.x; w < w1;
         w += (int64_t)gridDim.x * blockDim.x) {
        if (w == w0 && (old_nodes & 31)) legal[w] &= (1u << (old_nodes & 31)) - 1u;
        else legal[w] = 0u;
    }
}

// One wavefront per leaf.  The children are written first, the leaf's child range last: a
// node is a leaf exactly while its child count is 0.  The host offers no job for a leaf that
// already has children (the selection stopped at it because of the depth bound: it reads the
// child ranges first, so that such a leaf takes no ids); should one come all the same it is left
// alone.
__global__ __launch_bounds__(64) void k_expand(ForestMut f, const ExpandJob *jobs, int n_jobs, const int32_t *moves,
                                               const float *priors, int32_t *status) {
    const int j = blockIdx.x;
    if (j >= n_jobs) return;
    const ExpandJob job = jobs[j];
    const bool fresh = f.span[job.leaf].y == 0;
    for (int i = threadIdx.x; i < job.count; i += 64) {
        const int id = job.begin + i;
        f.N[id] = 0;
        f.W[id] = 0.0f;
        f.P[id] = fresh ? priors[job.off + i] : 0.0f;
        f.VL[id] = 0;
        if (f.rN) f.rN[id] = 0;
        if (f.rW) f.rW[id] = 0.0f;
        if (f.q2) f.q2[id] = 0.0f;  // getCombinedValue of a node without visits of either kind
        f.span[id] = int2{0, 0};
        if (f.action) f.action[id] = moves[job.off + i];
        if (f.hash) f.hash[id] = ~0ull;  // no position key yet (omk_forest_set_keys)
        if (f.legal && fresh) atomicOr(f.legal + ((uint32_t)id >> 5), 1u << ((uint32_t)id & 31u));
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        if (fresh) f.span[job.leaf] = int2{job.begin, job.count};
        status[j] = fresh ? job.begin : -1;
    }
}

hipError_t launch_expand(const ForestMut &f, const ExpandJob *jobs, int n_jobs, const int32_t *moves,
                         const float *priors, int32_t *status, int64_t old_nodes, int64_t new_nodes, hipStream_t s) {
    if (n_jobs <= 0) return hipSuccess;
    if (f.legal) hipLaunchKernelGGL(k_expand_mask, dim3(64), dim3(256), 0, s, f.legal, old_nodes, new_nodes);
    hipLaunchKernelGGL(k_expand, dim3(n_jobs), dim3(64), 0, s, f, jobs, n_jobs, moves, priors, status);
    return hipGetLastError();
}

// ---- RAVE statistics of MCTSEngine::backPropagate (src/mcts/mcts_engine_tree.cpp:288-331,
// MCTSNode::updateRAVE src/mcts/mcts_node.cpp:631-643): every child of a path node whose
// action occurs among the path's actions gets rN += 1, rW += the node's signed value ----
constexpr int kRaveMaxLen = 4097;  // longest path the ABI accepts

// One wavefront per (traversal, depth): the path's actions go to LDS, the node's children are
// spread over the lanes.
__global__ __launch_bounds__(64) void k_rave_backup(ForestMut f, const int32_t *paths, const int32_t *path_len,
                                                    const float *values, int n, int stride) {
    __shared__ int s_pa[kRaveMaxLen];
    const int t = blockIdx.x, d = blockIdx.y, lane = threadIdx.x;
    const int len = path_len[t];
    if (d >= len) return;
    const int node = paths[(size_t)d * stride + t];
    const int2 sp = f.span[node];
    if (sp.y <= 0) return;
    for (int e = lane; e < len; e += 64) {
        const int pn = paths[(size_t)e * stride + t];
        s_pa[e] = f.action ? f.action[pn] : pn;
    }
    __syncthreads();
    float v = values[t];
    if ((len - 1 - d) & 1) v = -v;  // the leaf's children see +value, every ply up flips it
    for (int i = lane; i < sp.y; i += 64) {
        const int id = sp.x + i;
        if (f.legal && !((f.legal[(uint32_t)id >> 5] >> ((uint32_t)id & 31u)) & 1u)) continue;
        const int a = f.action ? f.action[id] : id;
        bool hit = false;
        for (int e = 0; e < len && !hit; e++) hit = s_pa[e] != -1 && s_pa[e] == a;
        if (hit) {
            atomicAdd(f.rN + id, 1);
            unsafeAtomicAdd(f.rW + id, v);
        }
    }
}

hipError_t launch_rave_backup(const ForestMut &f, const int32_t *paths, const int32_t *path_len, const float *values,
                              int n, int stride, int max_len, hipStream_t s) {
    if (n <= 0 || max_len <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_rave_backup, dim3(n, max_len), dim3(64), 0, s, f, paths, path_len, values, n, stride);
    return hipGetLastError();
}

// ---- compaction after re-rooting: gathers through the old-id-of-new-id map ----
__global__ __launch_bounds__(256) void k_gather_words(uint32_t *dst, const uint32_t *src, const int32_t *map, int64_t k) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < k) dst[i] = src[map[i]];
}

__global__ __launch_bounds__(256) void k_gather_dwords(uint64_t *dst, const uint64_t *src, const int32_t *map,
                                                       int64_t k) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < k) dst[i] = src[map[i]];
}

__global__ __launch_bounds__(256) void k_gather_span(int2 *dst, const int2 *src, const int32_t *map,
                                                     const int32_t *new_begin, int64_t k) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < k) {
        const int cc = src[map[i]].y;
        dst[i] = int2{cc > 0 ? new_begin[i] : 0, cc};
    }
}

hipError_t launch_gather_words(uint32_t *dst, const uint32_t *src, const int32_t *map, int64_t k, hipStream_t s) {
    if (k <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_gather_words, dim3((unsigned)((k + 255) / 256)), dim3(256), 0, s, dst, src, map, k);
    return hipGetLastError();
}

hipError_t launch_gather_dwords(uint64_t *dst, const uint64_t *src, const int32_t *map, int64_t k, hipStream_t s) {
    if (k <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_gather_dwords, dim3((unsigned)((k + 255) / 256)), dim3(256), 0, s, dst, src, map, k);
    return hipGetLastError();
}

hipError_t launch_gather_span(int2 *dst, const int2 *src, const int32_t *map, const int32_t *new_begin, int64_t k,
                              hipStream_t s) {
    if (k <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_gather_span, dim3((unsigned)((k + 255) / 256)), dim3(256), 0, s, dst, src, map, new_begin, k);
    return hipGetLastError();
}

// plain copy of 4-byte words: the known-size kernel that hardware traffic counters are scaled by
__global__ __launch_bounds__(256) void k_copy_words(uint32_t *dst, const uint32_t *src, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * 256;
    for (; i < n; i += step) dst[i] = src[i];
}

hipError_t launch_copy_words(void *dst, const void *src, int64_t n_words, hipStream_t s) {
    if (n_words <= 0) return hipSuccess;
    int64_t blocks = (n_words + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(k_copy_words, dim3((unsigned)blocks), dim3(256), 0, s, (uint32_t *)dst, (const uint32_t *)src,
                       n_words);
    return hipGetLastError();
}

hipError_t launch_apply_vl(const ForestDev &f, const int32_t *paths, const int32_t *path_len, int n, int stride,
                           int max_len, int vl, hipStream_t s) {
    if (vl <= 0 || n <= 0 || max_len <= 1) return hipSuccess;
    hipLaunchKernelGGL(k_apply_vl, dim3((n + 255) / 256, max_len - 1), dim3(256), 0, s, f, paths, path_len, n,
                       stride, vl);
    return hipGetLastError();
}

hipError_t launch_revert_vl(const ForestDev &f, const int32_t *paths, const int32_t *path_len, int n, int stride,
                            int max_len, int vl, hipStream_t s) {
    if (vl <= 0 || n <= 0 || max_len <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_revert_vl, dim3((n + 255) / 256, max_len), dim3(256), 0, s, f, paths, path_len, n, stride,
                       vl);
    return hipGetLastError();
}

hipError_t launch_backup(const ForestDev &f, const int32_t *paths, const int32_t *path_len, const float *values,
                         int n, int stride, int max_len, int vl, hipStream_t s) {
    if (n <= 0 || max_len <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_backup, dim3((n + 255) / 256, max_len), dim3(256), 0, s, f, paths, path_len, values, n,
                       stride, vl);
    return hipGetLastError();
}

// ---- the RAVE blend kept per node ----
// MCTSNode::getCombinedValue (reference src/mcts/mcts_node.cpp:657-678) is a function of the node's own N, W,
// rN, rW and the RAVE constant; virtual loss does not enter.  A selection reads it for every child of every
// node visited (three divisions and a square root each), and between two backups it does not change: it is
// kept in f.q2, computed by the same function from the same binary32 inputs as the selection would, by
// whatever changes one of the four (upload, backup; a node created by an expansion starts at 0).
__global__ void k_blend_all(ForestDev f, float rave_k) {
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < f.n_nodes; i += (int64_t)gridDim.x * blockDim.x)
        f.q2[i] = combined_value(f.N[i], f.W[i], f.rN[i], f.rW[i], rave_k);
}

__global__ void k_blend_paths(ForestDev f, const int32_t *paths, const int32_t *path_len, int n, int stride,
                              float rave_k) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    const int d = blockIdx.y;
    if (t >= n || d >= path_len[t]) return;
    const int node = paths[(size_t)d * stride + t];
    if (node < 0 || node >= f.n_nodes) return;
    f.q2[node] = combined_value(f.N[node], f.W[node], f.rN[node], f.rW[node], rave_k);
}

hipError_t launch_blend_all(const ForestDev &f, float rave_k, hipStream_t s) {
    if (!f.q2 || f.n_nodes <= 0) return hipSuccess;
    const int64_t blocks = std::min<int64_t>((f.n_nodes + 255) / 256, 1 << 16);
    hipLaunchKernelGGL(k_blend_all, dim3((unsigned)blocks), dim3(256), 0, s, f, rave_k);
    return hipGetLastError();
}

hipError_t launch_blend_paths(const ForestDev &f, const int32_t *paths, const int32_t *path_len, int n, int stride,
                              int max_len, float rave_k, hipStream_t s) {
    if (!f.q2 || n <= 0 || max_len <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_blend_paths, dim3((n + 255) / 256, max_len), dim3(256), 0, s, f, paths, path_len, n, stride,
                       rave_k);
    return hipGetLastError();
}

hipError_t launch_export(const ForestDev &f, const int32_t *paths, const int32_t *path_len, int n, int stride,
                         int max_depth, int32_t *out_paths, int32_t *out_actions, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    int64_t total = (int64_t)n * (max_depth + 1);
    hipLaunchKernelGGL(k_export, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, f, paths, path_len, n,
                       stride, max_depth, out_paths, out_actions);
    return hipGetLastError();
}

hipError_t launch_leaf_keys(const ForestDev &f, const int32_t *paths, const int32_t *path_len, int n, int stride,
                            const uint64_t *piece, int cells, const uint64_t *player, const uint64_t *root_key,
                            const int32_t *root_player, uint64_t *out, int *d_status, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_leaf_keys, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, f, paths, path_len, n,
                       stride, piece, cells, player, root_key, root_player, out, d_status);
    return hipGetLastError();
}

// ---- open-addressing transposition table: 16-byte slots, linear probing ----

constexpr unsigned long long kTTEmpty = ~0ull;

__device__ __forceinline__ uint64_t tt_home(uint64_t key, int log2_slots) {
    return (key * 0x9E3779B97F4A7C15ull) >> (64 - log2_slots);
}

__global__ __launch_bounds__(256) void k_tt_clear(TTSlot *slots, TTMeta *meta, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    TTSlot e;
    e.key = kTTEmpty;
    e.node = -1;
    e.depth = 0;
    slots[i] = e;
    TTMeta m;
    m.visits = 0u;
    m.value = 0.0f;
    m.last_access = 0u;
    m.claim = 0x7FFFFFFF;
    meta[i] = m;
}

// ---- PHMapTranspositionTable::store (phmap_transposition_table.cpp:51-84) for a batch of entries,
// in three passes.  Entry i of the call has the time t0 + i.  Among the entries of one call that
// carry the same key only the first (lowest i) is stored, which is what the serial order gives for
// the reference's call sites (a node stored from the traversal has no visits, hence replacement
// score 0, and never replaces; the leaves expanded in one step are distinct).

// Pass 1: every entry finds the slot of its key, or claims an empty one, and bids for it with its index.
__global__ __launch_bounds__(256) void k_tt_store_claim(TTSlot *slots, TTMeta *meta, int log2_slots,
                                                        const uint64_t *keys, const int32_t *nodes, int64_t n,
                                                        int64_t *slot_of, int *d_status) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    slot_of[i] = -1;
    if (nodes[i] < 0) return;  // nothing to store for this entry (store(): if (!node) return)
    unsigned long long key = keys[i];
    if (key == kTTEmpty) {
        atomicAdd(d_status + 1, 1);
        return;
    }
    uint64_t mask = (1ull << log2_slots) - 1ull;
    uint64_t s = tt_home(key, log2_slots);
    for (uint64_t probe = 0; probe <= mask; probe++, s = (s + 1) & mask) {
        unsigned long long prev = atomicCAS(&slots[s].key, kTTEmpty, key);
        if (prev == kTTEmpty) slots[s].depth = INT32_MIN;  // claimed just now: no entry behind the key yet
        if (prev == kTTEmpty || prev == key) {
            atomicMin(&meta[s].claim, (int)i);
            slot_of[i] = (int64_t)s;
            return;
        }
    }
    atomicAdd(d_status, 1);
}

__device__ __forceinline__ float tt_replacement_score(uint32_t visits, float value, int depth, uint32_t now,
                                                      uint32_t last_access) {
    // Entry::getReplacementScore (include/mcts/phmap_transposition_table.h:68-72)
    float recency = 1.0f / (1.0f + (float)(now - last_access));
    float importance = (float)visits * (1.0f + value) * (1.0f + (float)depth);
    return recency * importance;
}

// Pass 2: the winner of every slot creates the entry (createEntry :202-216: visits and value of the
// node as they are now) or replaces the one that is there when its score is better by the threshold.
// d_status[2] duplicates dropped, [3] new entries, [4] replacements.
__global__ __launch_bounds__(256) void k_tt_store_apply(ForestDev f, TTSlot *slots, TTMeta *meta,
                                                        const int32_t *nodes, const int32_t *depths, int64_t n,
                                                        const int64_t *slot_of, uint32_t t0, float threshold,
                                                        int *d_status) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int64_t s = slot_of[i];
    if (s < 0) return;
    if (meta[s].claim != (int)i) {
        atomicAdd(d_status + 2, 1);
        return;
    }
    const int node = nodes[i];
    const int depth = (int)(uint16_t)(depths ? depths[i] : 0);  // Entry::depth is a uint16_t
    uint32_t visits = 0u;
    float value = 0.0f;
    if (node < f.n_nodes) {
        const int nv = f.N[node];
        visits = (uint32_t)nv;
        value = nv == 0 ? 0.0f : f.W[node] / (float)nv;  // MCTSNode::getValue, src/mcts/mcts_node.cpp:484-490
    }
    bool write = false;
    if (slots[s].depth == INT32_MIN) {
        write = true;
        atomicAdd(d_status + 3, 1);
    } else {
        const uint32_t now = t0 + (uint32_t)i;
        const float existing = tt_replacement_score(meta[s].visits, meta[s].value, slots[s].depth, now, meta[s].last_access);
        const float fresh = tt_replacement_score(visits, value, depth, now, 0u);
        if (fresh > existing * (1.0f + threshold)) {
            write = true;
            atomicAdd(d_status + 4, 1);
        }
    }
    if (write) {
        slots[s].node = node;
        slots[s].depth = depth;
        meta[s].visits = visits;
        meta[s].value = value;
        meta[s].last_access = 0u;  // a new Entry starts with last_access 0
    }
}

// Pass 3: the bids are withdrawn.
__global__ __launch_bounds__(256) void k_tt_store_reset(TTMeta *meta, const int64_t *slot_of, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int64_t s = slot_of[i];
    if (s >= 0) meta[s].claim = 0x7FFFFFFF;
}

hipError_t launch_tt_store(const ForestDev &f, TTSlot *slots, TTMeta *meta, int log2_slots, const uint64_t *keys,
                           const int32_t *nodes, const int32_t *depths, int64_t n, int64_t *slot_of, uint32_t t0,
                           float threshold, int *d_status, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    hipLaunchKernelGGL(k_tt_store_claim, grid, block, 0, s, slots, meta, log2_slots, keys, nodes, n, slot_of, d_status);
    hipLaunchKernelGGL(k_tt_store_apply, grid, block, 0, s, f, slots, meta, nodes, depths, n, slot_of, t0, threshold,
                       d_status);
    hipLaunchKernelGGL(k_tt_store_reset, grid, block, 0, s, meta, slot_of, n);
    return hipGetLastError();
}

// ---- the transposition-table part of the traversal loop (mcts_engine_batch_tree_simple.cpp:116-162)
// over the paths of a selection ----

// The key of the state after every step of every path, the node selected there and its depth, laid
// out in the order the serial loop visits them (traversal-major: entry t * max_depth + d - 1 for step
// d >= 1 of traversal t); node -1 where the path has no such step.  Keys: the forest's per-node
// position keys, or (piece != nullptr) the root state's key with the piece keys of the path's moves
// folded in, as in k_leaf_keys.  store_nodes receives the node where the reference stores it
// (its visit count is 0, :116) and -1 elsewhere.
__global__ __launch_bounds__(256) void k_step_keys(ForestDev f, const int32_t *paths, const int32_t *path_len, int n,
                                                   int stride, int max_depth, const uint64_t *piece, int cells,
                                                   const uint64_t *player, const uint64_t *root_key,
                                                   const int32_t *root_player, uint64_t *keys, int32_t *step_nodes,
                                                   int32_t *store_nodes, int32_t *depths, int *d_status) {
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= n) return;
    const int len = path_len[t];
    const int p0 = piece ? (root_player[t] & 1) : 0;
    uint64_t h = piece ? root_key[t] : 0ull;
    bool bad = false;
    for (int d = 1; d <= max_depth; d++) {
        const size_t e = (size_t)t * max_depth + (d - 1);
        int node = -1;
        uint64_t key = ~0ull;
        if (d < len && !bad) {
            node = paths[(size_t)d * stride + t];
            if (node < 0 || node >= f.n_nodes) {
                bad = true;
                node = -1;
            } else if (piece) {
                const int act = f.action ? f.action[node] : node;
                if (act < 0 || act >= cells) {
                    bad = true;
                    node = -1;
                } else {
                    h ^= piece[(size_t)((p0 + d - 1) & 1) * cells + act];
                    key = (d & 1) ? h ^ player[p0] ^ player[p0 ^ 1] : h;
                }
            } else {
                key = f.hash[node];
            }
        }
        keys[e] = key;
        step_nodes[e] = node;
        store_nodes[e] = node >= 0 && f.N[node] == 0 ? node : -1;
        depths[e] = d;
    }
    if (bad) atomicAdd(d_status + 5, 1);
}

// What the loop does with a lookup (:141-156): a node other than the selected one, with visits, is a
// transposition.  It is reported (hit[e] = that node, else -1), never followed.
__global__ __launch_bounds__(256) void k_tt_hits(ForestDev f, const int32_t *step_nodes, const int32_t *found, int64_t n,
                                                 int32_t *hit, int *d_status) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int fn = found[i], node = step_nodes[i];
    int out = -1;
    if (node >= 0 && fn >= 0 && fn != node && fn < f.n_nodes && f.N[fn] > 0) out = fn;
    if (hit) hit[i] = out;  // a caller that only wants the count passes no array
    if (out >= 0) atomicAdd(d_status + 6, 1);
}

hipError_t launch_step_keys(const ForestDev &f, const int32_t *paths, const int32_t *path_len, int n, int stride,
                            int max_depth, const uint64_t *piece, int cells, const uint64_t *player,
                            const uint64_t *root_key, const int32_t *root_player, uint64_t *keys, int32_t *step_nodes,
                            int32_t *store_nodes, int32_t *depths, int *d_status, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_step_keys, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, f, paths, path_len, n, stride,
                       max_depth, piece, cells, player, root_key, root_player, keys, step_nodes, store_nodes, depths,
                       d_status);
    return hipGetLastError();
}

hipError_t launch_tt_hits(const ForestDev &f, const int32_t *step_nodes, const int32_t *found, int64_t n, int32_t *hit,
                          int *d_status, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_tt_hits, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, f, step_nodes, found, n, hit,
                       d_status);
    return hipGetLastError();
}

// d_status[0] counts entries that found no slot, d_status[1] keys equal to the empty marker
__global__ __launch_bounds__(256) void k_tt_insert(TTSlot *slots, int log2_slots, const uint64_t *keys,
                                                   const int32_t *nodes, const int32_t *depths, int64_t n,
                                                   int *d_status) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    unsigned long long key = keys[i];
    if (key == kTTEmpty) {
        atomicAdd(d_status + 1, 1);
        return;
    }
    uint64_t mask = (1ull << log2_slots) - 1ull;
    uint64_t s = tt_home(key, log2_slots);
    for (uint64_t probe = 0; probe <= mask; probe++, s = (s + 1) & mask) {
        unsigned long long prev = atomicCAS(&slots[s].key, kTTEmpty, key);
        if (prev == kTTEmpty) {
            slots[s].node = nodes[i];
            slots[s].depth = depths ? depths[i] : 0;
            return;
        }
        if (prev == key) return;  // already present: the first entry stays
    }
    atomicAdd(d_status, 1);
}

// meta / t0: a successful lookup stamps the entry with its time (PHMapTranspositionTable::lookup,
// phmap_transposition_table.cpp:107: last_access = access_counter++); lookup i of a call has the time
// t0 + i, the latest wins.
__global__ __launch_bounds__(256) void k_tt_probe(const TTSlot *slots, int log2_slots, const uint64_t *keys,
                                                  const int32_t *leaf, const uint64_t *node_hash, int64_t n_nodes,
                                                  int64_t n, int min_depth, int32_t *out, TTMeta *meta, uint32_t t0) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool valid = i < n;
    unsigned long long key = kTTEmpty;
    if (valid) {
        if (keys) key = keys[i];
        // a traversal without a leaf finds nothing; never index the forest with an id it does not have
        else if (leaf[i] >= 0 && leaf[i] < n_nodes) key = node_hash[leaf[i]];
    }
    int found = -1;
    unsigned long long hit_slot = ~0ull;
    if (key != kTTEmpty) {
        uint64_t mask = (1ull << log2_slots) - 1ull;
        uint64_t s = tt_home(key, log2_slots);
        for (uint64_t probe = 0; probe <= mask; probe++, s = (s + 1) & mask) {
            // one 16-byte load per slot touched
            uint4 raw = *reinterpret_cast<const uint4 *>(slots + s);
            unsigned long long k = ((unsigned long long)raw.y << 32) | raw.x;
            if (k == key) {
                if ((int)raw.w >= min_depth) {
                    found = (int)raw.z;
                    hit_slot = s;
                }
                break;
            }
            if (k == kTTEmpty) break;
        }
    }
    if (meta) {
        // Thousands of traversals can end at one leaf (a crowd that follows one child all the way
        // down; a few hundred distinct leaves for 16384 traversals is typical), and atomics on
        // one address are served one by one: of the lookups of a wavefront that found the same
        // entry only the last, whose time is the latest, stamps it.
        const unsigned lane = threadIdx.x & 63u;
        unsigned long long todo = __ballot(hit_slot != ~0ull);
        while (todo) {
            const int lead = __ffsll((long long)todo) - 1;
            const unsigned long long s0 = __shfl(hit_slot, lead);
            const unsigned long long same = __ballot(hit_slot == s0);
            if (lane == 63u - (unsigned)__clzll((long long)same)) atomicMax(&meta[s0].last_access, t0 + (uint32_t)i);
            todo &= ~same;
        }
    }
    if (valid) out[i] = found;
}

// Position keys of single nodes, from the host's game states (IGameState::getHash of the state a
// node stands for).  An id outside the forest is counted, not written.
__global__ __launch_bounds__(256) void k_set_keys(uint64_t *hash, const int32_t *nodes, const uint64_t *keys, int64_t n,
                                                  int64_t n_nodes, int *d_bad) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int node = nodes[i];
    if (node < 0 || node >= n_nodes) {
        atomicAdd(d_bad, 1);
        return;
    }
    hash[node] = keys[i];
}

hipError_t launch_set_keys(uint64_t *hash, const int32_t *nodes, const uint64_t *keys, int64_t n, int64_t n_nodes,
                           int *d_bad, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_set_keys, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, hash, nodes, keys, n, n_nodes, d_bad);
    return hipGetLastError();
}

hipError_t launch_tt_clear(TTSlot *slots, TTMeta *meta, int log2_slots, hipStream_t s) {
    int64_t n = 1ll << log2_slots;
    hipLaunchKernelGGL(k_tt_clear, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, slots, meta, n);
    return hipGetLastError();
}

hipError_t launch_tt_probe(const TTSlot *slots, int log2_slots, const uint64_t *keys, const int32_t *leaf,
                           const uint64_t *node_hash, int64_t n_nodes, int64_t n, int min_depth, int32_t *out,
                           TTMeta *meta, uint32_t t0, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_tt_probe, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, slots, log2_slots, keys, leaf,
                       node_hash, n_nodes, n, min_depth, out, meta, t0);
    return hipGetLastError();
}

// ---- the traversal loop with the transposition table on, redirects included
// (reference src/mcts/mcts_engine_batch_tree_simple.cpp:88-165: store :116-128, lookup :131-141, redirect
// :142-156; MCTSNode::updateChildReference src/mcts/mcts_node.cpp:617-630) ----
//
// A redirect re-points a child slot of one node at a node that lives under another: the tree becomes a
// graph, a node's visitors no longer all come through one parent, and what a traversal finds depends on
// what every earlier one stored, found and re-pointed.  The reference's outcome for one thread is the
// outcome of the traversals run one after the other, and that is what this kernel does: ONE wavefront
// walks the traversals in index order, the children of a node spread over its lanes (64 slots a round),
// the table and the re-pointing done by lane 0.  It is the exact mode for a search that wants the
// reference's redirects, not a fast one: a step costs a few dependent trips to memory, and nothing
// overlaps them.
//
// alias[s] >= 0: child slot s holds that node instead of node s.  The statistics, the prior and the
// action that selection and the move record read are those of the node a slot HOLDS
// (children_[i]->getAction(), :112).  The key of a step is the position key of the node of the
// ORIGINAL tree (slots, not what they hold) that the recorded moves lead to from the root, which is
// what replaying the recorded moves on the root state gives (:119-124, :133-137); where no such node
// exists the step has no key and the table is left alone.
// Time: the reference's access counter as one thread advances it, from t0 on: it ticks on a store that
// finds its key (phmap_transposition_table.cpp:65) and on a lookup that hits (:107), not otherwise.

__device__ __forceinline__ int ld_agent(const int32_t *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ bool slot_legal(const ForestDev &f, int id) {
    return !f.legal || ((f.legal[(uint32_t)id >> 5] >> ((uint32_t)id & 31u)) & 1u);
}

// MCTSNode::selectChild over the slots [cb, cb + cc) of `node`; returns the chosen slot or -1.  The
// same arithmetic (child_keys) and the same choice as the tree kernels: the first maximum of the first
// scan, a second-scan candidate only when it beats every score before it and only after a first scan
// that found a child, the least visited child when no score is real.
template <bool RAVE>
__device__ __forceinline__ int pick_slot_redirected(const ForestDev &f, const int32_t *alias, int node, int cb, int cc,
                                                    float c_puct, float rave_k, int lane) {
    const float ep = c_puct * sqrtf((float)f.N[node]);
    uint32_t b1 = 0u, p1 = 0xFFFFFFFFu, b2 = 0u, p2 = 0xFFFFFFFFu, fn = 0xFFFFFFFFu, fi = 0xFFFFFFFFu;
    for (int base = 0; base < cc; base += kWave) {
        const int i = base + lane;
        const bool in = i < cc && slot_legal(f, cb + i);
        if (in) {
            const int al = ld_agent(alias + cb + i);
            const int held = al >= 0 ? al : cb + i;
            const int n = f.N[held];
            const float w = f.W[held];
            const int vl = ld_agent(f.VL + held);
            float q2 = 0.0f;
            if (RAVE) q2 = combined_value(n, w, f.rN[held], f.rW[held], rave_k);
            uint32_t k1, k2;
            child_keys<RAVE>(n, w, f.P[held], vl, q2, ep, k1, k2);
            if (k1 > b1) { b1 = k1; p1 = (uint32_t)i; }
            if (k2 > b2) { b2 = k2; p2 = (uint32_t)i; }
            const uint32_t on = (uint32_t)n ^ 0x80000000u;
            if (on < fn) { fn = on; fi = (uint32_t)i; }
        }
    }
    const uint32_t m1 = wave_max_u32(b1);
    if (m1 != 0u) {
        const uint32_t m2 = wave_max_u32(b2);
        if (m2 > m1) return cb + (int)wave_min_u32(b2 == m2 ? p2 : 0xFFFFFFFFu);
        return cb + (int)wave_min_u32(b1 == m1 ? p1 : 0xFFFFFFFFu);
    }
    const uint32_t gm = wave_min_u32(fn);
    const uint32_t idx = wave_min_u32(fn == gm ? fi : 0xFFFFFFFFu);
    return idx == 0xFFFFFFFFu ? -1 : cb + (int)idx;
}

// The winning slot of one round of candidates (see pick_slot_redirected): index among the slots, or ~0.
__device__ __forceinline__ uint32_t pick_of_round(uint32_t b1, uint32_t p1, uint32_t b2, uint32_t p2, uint32_t fn,
                                                 uint32_t fi) {
    const uint32_t m1 = wave_max_u32(b1);
    if (m1 != 0u) {
        const uint32_t m2 = wave_max_u32(b2);
        if (m2 > m1) return wave_min_u32(b2 == m2 ? p2 : 0xFFFFFFFFu);
        return wave_min_u32(b1 == m1 ? p1 : 0xFFFFFFFFu);
    }
    const uint32_t gm = wave_min_u32(fn);
    return wave_min_u32(fn == gm ? fi : 0xFFFFFFFFu);
}

// A step is a chain of dependent trips to memory and nothing overlaps them, so the walk asks for as much as it
// can in one trip.  A node of at most 64 slots (one per lane): alias, legality word, statistics, action, position
// key and child range of every slot come together, read as if no slot were re-pointed; the few lanes whose slot
// IS re-pointed read their node's again.  What the step needs next is then in registers: the chosen node's
// visit count (the next node's N_parent, and the store's "no visits yet"), its action, its child range, and,
// while the recorded moves still lead along the nodes walked (shadow == cur), the key of the position reached,
// which is the key of the slot that carries the recorded move.  Two dependent trips a step are left: the
// children, then the table's slot.  Wider nodes and paths whose recorded moves have left the nodes walked take
// the plain sequence of loads.
template <bool RAVE>
__global__ __launch_bounds__(kWave) void k_select_redirect(ForestDev f, RedirectArgs a) {
    const int lane = threadIdx.x;
    const uint64_t mask = (1ull << a.log2_slots) - 1ull;
    int n_new = 0, n_repl = 0, n_found = 0, n_redirect = 0, n_full = 0, n_trunc = 0;
    uint32_t g = 0u;
    uint32_t clk = a.t0;  // the table's access counter (lane 0 keeps it)
    for (int t = 0; t < a.n; t++) {
        int cur = a.paths[t];
        int shadow = cur;
        int d = 0;
        int2 sp = f.span[cur];
        int np = f.N[cur];
        for (;;) {
            int slot = -1, best = -1, nbest = 0, move = 0, shadow_next = -1;
            int2 nsp = int2{0, 0};
            unsigned long long key = kTTEmpty;
            bool key_known = false;
            if (sp.y > 0 && d < a.max_depth) {
                if (sp.y <= kWave) {
                    const int s = sp.x + lane;
                    const bool in_range = lane < sp.y;
                    uint32_t word = 0xFFFFFFFFu;
                    int al = -1, n = 0, vl = 0, act = s, rn = 0;
                    float w = 0.0f, p = 0.0f, rw = 0.0f;
                    int2 csp = int2{0, 0};
                    unsigned long long hk = kTTEmpty;
                    if (in_range) {
                        if (f.legal) word = f.legal[(uint32_t)s >> 5];
                        al = ld_agent(a.alias + s);
                        n = f.N[s];
                        w = f.W[s];
                        p = f.P[s];
                        vl = ld_agent(f.VL + s);
                        if (f.action) act = f.action[s];
                        hk = f.hash[s];
                        csp = f.span[s];
                        if (RAVE) {
                            rn = f.rN[s];
                            rw = f.rW[s];
                        }
                    }
                    const bool in = in_range && ((word >> ((uint32_t)s & 31u)) & 1u);
                    const int act_slot = act;  // the move this slot stands for in the tree as uploaded
                    int held = s;
                    if (in && al >= 0) {  // a re-pointed slot: the node it holds
                        held = al;
                        n = f.N[held];
                        w = f.W[held];
                        p = f.P[held];
                        vl = ld_agent(f.VL + held);
                        act = f.action ? f.action[held] : held;
                        csp = f.span[held];
                        if (RAVE) {
                            rn = f.rN[held];
                            rw = f.rW[held];
                        }
                    }
                    uint32_t k1 = 0u, k2 = 0u, on = 0xFFFFFFFFu;
                    if (in) {
                        const float q2 = RAVE ? combined_value(n, w, rn, rw, a.rave_k) : 0.0f;
                        child_keys<RAVE>(n, w, p, vl, q2, a.c_puct * sqrtf((float)np), k1, k2);
                        on = (uint32_t)n ^ 0x80000000u;
                    }
                    const uint32_t idx = pick_of_round(k1, (uint32_t)lane, k2, (uint32_t)lane, on, in ? (uint32_t)lane : 0xFFFFFFFFu);
                    if (idx != 0xFFFFFFFFu) {
                        const int L = (int)idx;
                        slot = sp.x + L;
                        best = __builtin_amdgcn_readlane(held, L);
                        nbest = __builtin_amdgcn_readlane(n, L);
                        move = __builtin_amdgcn_readlane(act, L);
                        nsp.x = __builtin_amdgcn_readlane(csp.x, L);
                        nsp.y = __builtin_amdgcn_readlane(csp.y, L);
                        if (shadow == cur) {
                            const unsigned long long any = __ballot(in && act_slot == move);
                            if (any) {
                                const int l2 = __ffsll((long long)any) - 1;
                                shadow_next = sp.x + l2;
                                const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)hk, l2);
                                const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(hk >> 32), l2);
                                key = ((unsigned long long)hi << 32) | lo;
                            }
                            key_known = true;
                        }
                    }
                } else {
                    slot = pick_slot_redirected<RAVE>(f, a.alias, cur, sp.x, sp.y, a.c_puct, a.rave_k, lane);
                    if (slot >= 0) {
                        const int al = ld_agent(a.alias + slot);
                        best = al >= 0 ? al : slot;
                        nbest = f.N[best];
                        move = f.action ? f.action[best] : best;
                        nsp = f.span[best];
                    }
                }
            }
            if (slot < 0) {
                if (lane == 0) {
                    a.leaf[t] = cur;
                    a.path_len[t] = d + 1;
                }
                if (sp.y > 0 && d >= a.max_depth) n_trunc++;
                break;
            }
            if (!key_known) {
                if (shadow >= 0) {
                    const int2 ss = f.span[shadow];
                    for (int base = 0; base < ss.y && shadow_next < 0; base += kWave) {
                        const int i = base + lane;
                        const int s = ss.x + i;
                        const bool hit = i < ss.y && slot_legal(f, s) && (f.action ? f.action[s] : s) == move;
                        const unsigned long long any = __ballot(hit);
                        if (any) shadow_next = ss.x + base + (__ffsll((long long)any) - 1);
                    }
                }
                if (shadow_next >= 0) key = f.hash[shadow_next];
            }
            int redirected = 0;
            if (lane == 0) {
                if (a.vl > 0) atomicAdd(f.VL + best, a.vl);                       // :109
                if (a.moves) a.moves[(size_t)d * a.stride + t] = move;            // :112
                if (key != kTTEmpty) {
                    uint64_t s = tt_home(key, a.log2_slots);
                    uint64_t probe = 0;
                    for (; probe <= mask; probe++, s = (s + 1) & mask) {
                        const unsigned long long k = a.slots[s].key;
                        if (k == key || k == kTTEmpty) break;
                    }
                    const bool room = probe <= mask;
                    const bool present = room && a.slots[s].key == key;
                    if (nbest == 0) {                                             // :116-128, store()
                        if (!room) {
                            n_full++;
                        } else {
                            const int depth = (int)(uint16_t)(d + 1);             // move_sequence.size(); Entry::depth is a uint16_t
                            bool write = !present;
                            if (present) {
                                const uint32_t now = clk++;                       // :65
                                const float existing = tt_replacement_score(a.meta[s].visits, a.meta[s].value, a.slots[s].depth,
                                                                            now, a.meta[s].last_access);
                                const float fresh = tt_replacement_score(0u, 0.0f, depth, now, 0u);
                                if (fresh > existing * (1.0f + a.threshold)) {
                                    write = true;
                                    n_repl++;
                                }
                            } else {
                                n_new++;
                            }
                            if (write) {
                                a.slots[s].key = key;
                                a.slots[s].node = best;
                                a.slots[s].depth = depth;
                                a.meta[s].visits = 0u;
                                a.meta[s].value = 0.0f;
                                a.meta[s].last_access = 0u;
                            }
                        }
                    }
                    int found = -1;
                    if (room && a.slots[s].key == key) {                          // :141, lookup()
                        found = a.slots[s].node;
                        a.meta[s].last_access = clk++;                            // :107
                        n_found++;
                    }
                    if (found >= 0 && found != best && found < f.n_nodes && f.N[found] > 0) {   // :142
                        if (a.vl > 0) {
                            vl_sub_clamp(f.VL + best, a.vl);                      // :146
                            atomicAdd(f.VL + found, a.vl);                        // :152
                        }
                        // :149: the slot selected is the first slot of the node that holds the old child (two slots
                        // holding one node score alike, and the first of equals is selected)
                        __hip_atomic_store(a.alias + slot, found, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        best = found;
                        redirected = 1;
                        n_redirect++;
                    }
                }
                a.paths[(size_t)(d + 1) * a.stride + t] = best;
            }
            best = __builtin_amdgcn_readfirstlane(best);
            redirected = __builtin_amdgcn_readfirstlane(redirected);
            // what lane 0 wrote is what every lane reads from here on: one wavefront, whose accesses to an address
            // reach the cache in program order; virtual loss and aliases are read past the first-level cache
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            if (redirected) {
                nsp = f.span[best];
                nbest = f.N[best];
            }
            cur = best;
            sp = nsp;
            np = nbest;
            shadow = shadow_next;
            d++;
            g++;
        }
    }
    if (lane == 0) {
        a.counts[0] = n_new;
        a.counts[1] = n_repl;
        a.counts[2] = n_found;
        a.counts[3] = n_redirect;
        a.counts[4] = (int)g;
        a.counts[5] = n_full;
        a.counts[6] = (int)(clk - a.t0);
        *a.truncated = n_trunc;
        *a.truncated_next = 0;
        *a.abort_word = 0;
    }
}

hipError_t launch_select_redirect(const ForestDev &f, const RedirectArgs &a, bool rave, hipStream_t s) {
    if (rave) hipLaunchKernelGGL(k_select_redirect<true>, dim3(1), dim3(kWave), 0, s, f, a);
    else hipLaunchKernelGGL(k_select_redirect<false>, dim3(1), dim3(kWave), 0, s, f, a);
    return hipGetLastError();
}

hipError_t launch_tt_insert(TTSlot *slots, int log2_slots, const uint64_t *keys, const int32_t *nodes,
                            const int32_t *depths, int64_t n, int *d_status, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_tt_insert, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, slots, log2_slots, keys,
                       nodes, depths, n, d_status);
    return hipGetLastError();
}

}  // namespace omk
