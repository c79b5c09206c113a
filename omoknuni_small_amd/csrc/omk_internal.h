// Internal declarations shared by the translation units of libomk_forest.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "omk_device.h"

namespace omk {

// Per-node arrays in HBM (structure of arrays; siblings are contiguous in every array).
struct ForestDev {
    const int2 *span;  // (child_begin, child_count); child_count 0 = not expanded
    int32_t *N;
    float *W;
    const float *P;
    int32_t *VL;
    const int32_t *rN;
    const float *rW;
    // RAVE blend of every node (MCTSNode::getCombinedValue: a function of the node's own N, W, rN, rW and the
    // RAVE constant, not of virtual loss), kept by whatever changes these four; nullptr without RAVE arrays
    float *q2;
    const uint32_t *legal;  // nullptr = every slot holds a child
    const int32_t *action;  // nullptr = node id
    const uint64_t *hash;   // nullptr = none
    int64_t n_nodes;
};

// A node together with the traversals that reached it: seg[off .. off+m) holds their
// indices in ascending order.  np is the node's visit count as read by the parent's wave.
struct Item {
    int32_t node;
    int32_t off;    // first entry of its visitor list (single-visitor queue: the traversal itself)
    int32_t m;      // visitors
    int32_t np;     // N(node) as read by the parent's wavefront
    int32_t depth;  // depth of the node on the visitors' paths
    int32_t pad[3]; // [0] 0 = node, 1 = slice of a heavy node, 2 = part of its partition, 3 = node whose visitor
                    // list is still being written, 4 = one boundary of a node to work out ahead of time;
                    // [1] context; [2] slice | slices << 16 (kind 4: boundary | slice size << 8)
};

constexpr int kHeavyCtxInts = 16 + 1024;  // 16 + the widest fan-out
constexpr int kHeavyMin = 1024;          // visitors from which a node is settled by several wavefronts
constexpr int kMaxSlices = 64;           // slices (and parts of the partition) of such a node, at most
constexpr int kHeavyFanout = 384;        // widest node settled that way (register budget)
constexpr int kSliceEntries = 192;       // visitors per slice of such a node, about
// Visitors per slice of a heavy node: a function of the visitor count in steps (kSliceEntries up to
// kSliceEntries * kMaxSlices visitors, then the next multiple of 64 that keeps the slices at kMaxSlices), so that
// whoever knows the count only within a step knows the slice size.  (128 visitors a slice and up to 128 slices
// measured the same as 192 and 64: a slice's time is mostly not its entries.)
__host__ __device__ inline int slice_size(int m) {
    const int s = ((m + 64 * kMaxSlices - 1) / (64 * kMaxSlices)) << 6;
    return s < kSliceEntries ? kSliceEntries : s;
}

// The boundaries between the slices of a heavy node: whoever needs one first works it out and leaves it here.
// Per boundary: [0] 2 * the number of the select call while it is being worked out, that + 1 once the rest is
// written, [1] the threshold key, [2] entries above the boundary, [3] 1 = worked out, 0 = the threshold search
// failed, [16 + i] entries of child i above the boundary.
constexpr int kBoundInts = 16 + kHeavyFanout;

struct SelectArgs {
    const Item *items0;    // level-0 items with several visitors, built when the roots are set
    const int32_t *seg0;   // their visitor lists
    const Item *singles0;  // traversals alone at their root: (node, traversal, depth 0, -)
    Item *singles_q;       // single visitors: (node, traversal, depth, N of the node)
    int32_t *n_singles;
    Item *items_q;         // multi-visitor work queue, q_cap slots, filled front to back
    int32_t *q_ready;      // per slot: == epoch once the item and everything it refers to is written
    // Scheduler words, each on a memory line (and channel) of its own: waiting wavefronts
    // poll sched_wait, working wavefronts bump the others, and neither queues behind the other.
    int32_t *sched_head;   // next ticket
    int32_t *sched_tail;   // slots handed out
    int32_t *sched_wait;   // [0] visitors still in multi-visitor items, [1] abort flag (a waiting
                           // wavefront gave up, or the queue overflowed)
    int32_t *hctx;         // contexts of heavy nodes, kHeavyCtxInts each: [0] slices still running,
                           // [1] a slice failed a check, [5] == the number of the select call when the contexts of
                           // children are listed, [16 + i] visits of child i, [16 + kHeavyFanout + i] context + 1
                           // of child i whose boundaries are being worked out ahead of time, or 0
    int32_t *hctx_n;       // contexts handed out
    int32_t *hbound;       // boundaries between the slices of heavy nodes: kMaxSlices x kBoundInts per context
    int32_t *list_flag;    // per visitor-list start: depth of the deepest item whose list, starting there,
                           // is complete (items of kind 3 are published before their list is written)
    int32_t hctx_cap;
    int32_t poll_sleep;    // s_sleep(32) units between two polls of a waiting wavefront
    int32_t q_cap;
    int32_t epoch;         // number of this select call on the batch, > 0
    long long *trace;      // nullptr, or per processed node: start, end (100 MHz clock), visitors | depth << 32 |
                           // kind << 60, node | number << 32, and eight words (what a slice of a heavy node did)
    int32_t *trace_n;
    int32_t trace_cap;
    int32_t *times;        // [0] when the first block of the persistent launch started, [1] when the last team
                           // left, [2] when the last walker left (100 MHz clock, low 31 bits)
    int32_t spin_limit;    // polls of a waiting wavefront before it raises the abort flag
    int32_t *single_ready;  // per entry of the single-visitor queue: number of the select call that wrote it
    int32_t *singles_head;  // tickets of the walkers of the persistent launch
    int32_t n_trav;         // traversals of the batch (entries the single-visitor queue can hold)
    int32_t n_team_blocks;  // blocks of the persistent launch that are teams; the blocks behind them are walkers
    int32_t fast_singles;   // the walkers use the variant of select_single that trades bytes for latency
    int32_t *seg[2];       // visitor lists of level L >= 1 live in seg[(L-1)&1]
    int32_t *sc_child;     // per visitor: chosen child index (two halves of `stride`, alternating with the depth)
    int32_t *sc_occ;       // per visitor: how many earlier visitors of the item chose the same child
    int32_t *paths;        // level-major [max_depth+1][stride]
    int32_t *path_len;
    int32_t *leaf;
    int32_t *truncated;       // simulations cut by max_depth in this select: zero when it starts ...
    int32_t *truncated_next;  // ... because the select before it cleared it: the counter of the next select
    int32_t *stats;        // optional 8 counters describing how the work was done (nullptr = off)
    int32_t stride;
    int32_t max_depth;
    int32_t vl;
    int32_t pw;
    float c_puct;
    float rave_k;
};

hipError_t launch_select(const ForestDev &f, const SelectArgs &a, int n_items0, int n_singles0, int n_traversals,
                         int max_fanout, bool rave, int n_cus, int n_hctx0, hipStream_t s);

hipError_t launch_apply_vl(const ForestDev &f, const int32_t *paths, const int32_t *path_len, int n, int stride,
                           int max_len, int vl, hipStream_t s);
hipError_t launch_revert_vl(const ForestDev &f, const int32_t *paths, const int32_t *path_len, int n, int stride,
                            int max_len, int vl, hipStream_t s);
hipError_t launch_backup(const ForestDev &f, const int32_t *paths, const int32_t *path_len, const float *values,
                         int n, int stride, int max_len, int vl, hipStream_t s);
// The per-node RAVE blend f.q2 from the node's statistics as they are: of every node, or of the nodes on the
// paths given (after a backup has changed their N and W).
hipError_t launch_blend_all(const ForestDev &f, float rave_k, hipStream_t s);
hipError_t launch_blend_paths(const ForestDev &f, const int32_t *paths, const int32_t *path_len, int n, int stride,
                              int max_len, float rave_k, hipStream_t s);
// row-major copies for the host: paths [n][max_depth+1], actions [n][max_depth], -1 padded
hipError_t launch_export(const ForestDev &f, const int32_t *paths, const int32_t *path_len, int n, int stride,
                         int max_depth, int32_t *out_paths, int32_t *out_actions, hipStream_t s);

hipError_t launch_leaf_keys(const ForestDev &f, const int32_t *paths, const int32_t *path_len, int n, int stride,
                            const uint64_t *piece, int cells, const uint64_t *player, const uint64_t *root_key,
                            const int32_t *root_player, uint64_t *out, int *d_status, hipStream_t s);
hipError_t launch_copy_words(void *dst, const void *src, int64_t n_words, hipStream_t s);
hipError_t launch_fill_words(void *dst, uint32_t value, int64_t n_words, hipStream_t s);
hipError_t launch_set_keys(uint64_t *hash, const int32_t *nodes, const uint64_t *keys, int64_t n, int64_t n_nodes,
                           int *d_bad, hipStream_t s);

// The same arrays for the one operation that writes the structure (leaf expansion).
struct ForestMut {
    int2 *span;
    int32_t *N;
    float *W;
    float *P;
    int32_t *VL;
    int32_t *rN;
    float *rW;
    float *q2;
    uint32_t *legal;
    int32_t *action;
    uint64_t *hash;
};

// One leaf to expand: its children get the ids [begin, begin + count) and the moves / priors
// moves[off .. off + count), priors[off .. off + count).
struct ExpandJob {
    int32_t leaf;
    int32_t begin;
    int32_t count;
    int32_t off;
};

hipError_t launch_expand(const ForestMut &f, const ExpandJob *jobs, int n_jobs, const int32_t *moves,
                         const float *priors, int32_t *status, int64_t old_nodes, int64_t new_nodes, hipStream_t s);

hipError_t launch_rave_backup(const ForestMut &f, const int32_t *paths, const int32_t *path_len, const float *values,
                              int n, int stride, int max_len, hipStream_t s);

// Compaction: new node i takes the statistics of old node map[i]; its child range keeps its
// length and starts at new_begin[i].
// Breadth-first renumbering of a subtree, level by level (omk_compact.hip).
hipError_t bfs_scan_bytes(int64_t max_items, size_t *bytes);
hipError_t launch_bfs_level(const int2 *span, int32_t *order, int32_t *new_begin, int64_t lo, int64_t cnt,
                            int64_t room, int32_t *cc, int32_t *scan, void *temp, size_t temp_bytes,
                            int64_t *h_total, hipStream_t s);
hipError_t launch_gather_legal(uint32_t *dst, const uint32_t *src, const int32_t *order, int64_t k, hipStream_t s);
hipError_t launch_gather_words(uint32_t *dst, const uint32_t *src, const int32_t *map, int64_t k, hipStream_t s);
hipError_t launch_gather_dwords(uint64_t *dst, const uint64_t *src, const int32_t *map, int64_t k, hipStream_t s);
hipError_t launch_gather_span(int2 *dst, const int2 *src, const int32_t *map, const int32_t *new_begin, int64_t k,
                              hipStream_t s);

struct TTSlot {
    unsigned long long key;
    int32_t node;
    int32_t depth;
};
// What PHMapTranspositionTable::Entry keeps beside key, node and depth for its replacement policy
// (include/mcts/phmap_transposition_table.h:48-72), in an array beside the slots: a probe reads
// the 16-byte slot only.
struct TTMeta {
    uint32_t visits;
    float value;
    uint32_t last_access;
    int32_t claim;  // lowest index of the entries of a store call that want this slot (0x7FFFFFFF between calls)
};
hipError_t launch_tt_clear(TTSlot *slots, TTMeta *meta, int log2_slots, hipStream_t s);
// d_status: [0] no free slot, [1] key equal to the empty marker, [2] duplicates of a key dropped,
// [3] new entries, [4] replacements, [5] paths with a step that has no key, [6] transpositions found
hipError_t launch_tt_store(const ForestDev &f, TTSlot *slots, TTMeta *meta, int log2_slots, const uint64_t *keys,
                           const int32_t *nodes, const int32_t *depths, int64_t n, int64_t *slot_of, uint32_t t0,
                           float threshold, int *d_status, hipStream_t s);
hipError_t launch_step_keys(const ForestDev &f, const int32_t *paths, const int32_t *path_len, int n, int stride,
                            int max_depth, const uint64_t *piece, int cells, const uint64_t *player,
                            const uint64_t *root_key, const int32_t *root_player, uint64_t *keys, int32_t *step_nodes,
                            int32_t *store_nodes, int32_t *depths, int *d_status, hipStream_t s);
hipError_t launch_tt_hits(const ForestDev &f, const int32_t *step_nodes, const int32_t *found, int64_t n, int32_t *hit,
                          int *d_status, hipStream_t s);
// The traversal loop with the table on, redirects included, one traversal after the other (omk_backup.hip).
struct RedirectArgs {
    int32_t *alias;
    TTSlot *slots;
    TTMeta *meta;
    int log2_slots;
    uint32_t t0;
    float threshold;
    int32_t *paths;     // level-major [max_depth + 1][stride]; level 0 holds the roots
    int32_t *path_len;
    int32_t *leaf;
    int32_t *moves;     // nullptr, or level-major [max_depth][stride]: the move recorded at every step
    int n, stride, max_depth, vl;
    float c_puct, rave_k;
    int *counts;        // [0] new entries, [1] replacements, [2] lookups that found an entry, [3] redirects,
                        // [4] steps, [5] stores that found the table full
    int32_t *truncated, *truncated_next, *abort_word;
};
hipError_t launch_select_redirect(const ForestDev &f, const RedirectArgs &a, bool rave, hipStream_t s);
// d_status[0] += entries that found no free slot, d_status[1] += keys equal to the empty marker
hipError_t launch_tt_insert(TTSlot *slots, int log2_slots, const uint64_t *keys, const int32_t *nodes,
                            const int32_t *depths, int64_t n, int *d_status, hipStream_t s);
// keys == nullptr: the key of entry i is node_hash[leaf[i]] (nothing for a leaf outside [0, n_nodes))
hipError_t launch_tt_probe(const TTSlot *slots, int log2_slots, const uint64_t *keys, const int32_t *leaf,
                           const uint64_t *node_hash, int64_t n_nodes, int64_t n, int min_depth, int32_t *out,
                           TTMeta *meta, uint32_t t0, hipStream_t s);

}  // namespace omk
