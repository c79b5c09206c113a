/*
 * ref_ptr -- the checker's arithmetic over the reference's DATA LAYOUT and threading, for
 * the timed CPU baseline.
 *
 * TEST INFRASTRUCTURE ONLY (like ref_cpu): only the benchmark's cpu_baseline leg and the
 * tests use it; nothing in the shipped library calls, links or loads it.
 *
 * What it restates (paths relative to the reference checkout):
 *   node record     include/mcts/mcts_node.h:154-178: children as a vector of shared
 *                   pointers, the five statistics as atomics on a cache line each, the prior
 *                   a plain float
 *   select_child    src/mcts/mcts_node.cpp:90-236 (two scans, strict >, first maximum), the
 *                   blend of :657-678, same operation order as ref_cpu.c
 *   traversal       src/mcts/mcts_engine_batch_tree_simple.cpp:73-185: an OpenMP loop over the
 *                   traversals, schedule(dynamic, 1), virtual loss added to every selected child
 *   backup          :276-281: update, revert the virtual loss, flip the sign, leaf to root
 *   virtual loss    src/mcts/mcts_node_virtual_loss.cpp:15-71 (fetch_add / fetch_sub + clamp,
 *                   compare-exchange loop on the value sum)
 *
 * With one thread the traversals run in index order and the paths are those of ref_cpu
 * (tests/test_oracle_ptr.py checks it); with several threads the result depends on the
 * schedule, as the reference's does, and only the time is used.
 *
 * Masked child slots of the dense board layouts do not exist in this flavour (the
 * reference creates children for legal moves only); the selection-time progressive
 * widening of the synthetic chess-like workload takes the first ceil(sqrt(N_parent))
 * children (prior-sorted storage), as ref_cpu does.
 */
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <memory>
#include <vector>

#include <omp.h>

namespace {

struct PNode {
    std::vector<std::shared_ptr<PNode>> children;
    int action = -1;
    int id = 0;
    float prior = 0.0f;
    alignas(64) std::atomic<int> visit_count{0};
    alignas(64) std::atomic<float> value_sum{0.0f};
    alignas(64) std::atomic<int> virtual_loss_count{0};
    alignas(64) std::atomic<int> rave_count{0};
    alignas(64) std::atomic<float> rave_value_sum{0.0f};
};

struct PTree {
    std::vector<std::shared_ptr<PNode>> nodes;  // by node id (owning, like the reference's parents)
    bool has_rave = false;
};

struct Params {
    float c_puct;
    int virtual_loss;
    int use_rave;
    float rave_k;
    int pw;
    int max_depth;
};

int ceil_sqrt(int n) {
    if (n <= 1) return 1;
    long long k = (long long)std::sqrt((double)n);
    while (k * k < (long long)n) k++;
    while ((k - 1) * (k - 1) >= (long long)n) k--;
    return (int)k;
}

float combined_value(const PNode &c, float rave_k) {
    const int visits = c.visit_count.load(std::memory_order_relaxed);
    const int rave_visits = c.rave_count.load(std::memory_order_relaxed);
    if (visits == 0 && rave_visits == 0) return 0.0f;
    const float mcts_value = visits > 0 ? c.value_sum.load(std::memory_order_relaxed) / (float)visits : 0.0f;
    const float rave_value =
        rave_visits > 0 ? c.rave_value_sum.load(std::memory_order_relaxed) / (float)rave_visits : 0.0f;
    const int three_v = (int)(3u * (uint32_t)visits);
    const float beta = std::sqrt(rave_k / ((float)three_v + rave_k));
    const float a = (1.0f - beta) * mcts_value;
    const float b = beta * rave_value;
    return a + b;
}

// the two scores a child shows: first scan and second scan
void child_scores(const PNode &c, float exploration_param, const Params &p, float &first, float &second) {
    const int child_visits = c.visit_count.load(std::memory_order_relaxed);
    const float child_value = c.value_sum.load(std::memory_order_relaxed);
    const int virtual_losses = c.virtual_loss_count.load(std::memory_order_relaxed);
    const int effective_visits = (int)((uint32_t)child_visits + (uint32_t)virtual_losses);
    const float effective_value = child_value - (float)virtual_losses;
    const float exploitation = effective_visits > 0 ? effective_value / (float)effective_visits : 0.0f;
    const float prod = c.prior * exploration_param;
    const float exploration = prod / (1.0f + (float)effective_visits);
    first = exploitation + exploration;
    const float exploitation2 = p.use_rave ? combined_value(c, p.rave_k) : exploitation;
    const int one_plus = (int)(1u + (uint32_t)effective_visits);
    second = exploitation2 + prod / (float)one_plus;
}

PNode *select_child(PNode &node, const Params &p) {
    const int parent_visits = node.visit_count.load(std::memory_order_relaxed);
    const float exploration_param = p.c_puct * std::sqrt((float)parent_visits);
    int count = (int)node.children.size();
    if (p.pw) {
        const int k = ceil_sqrt(parent_visits);
        if (k < count) count = k;
    }
    float best_score = -INFINITY;
    int best = -1;
    for (int i = 0; i < count; i++) {
        float s1, s2;
        child_scores(*node.children[i], exploration_param, p, s1, s2);
        if (s1 > best_score) {
            best_score = s1;
            best = i;
        }
    }
    if (best < 0 && count > 0) {
        int min_visits = INT32_MAX;
        for (int i = 0; i < count; i++) {
            const int v = node.children[i]->visit_count.load(std::memory_order_relaxed);
            if (v < min_visits) {
                min_visits = v;
                best = i;
            }
        }
    } else if (best >= 0) {
        for (int i = 0; i < count; i++) {
            float s1, s2;
            child_scores(*node.children[i], exploration_param, p, s1, s2);
            if (s2 > best_score) {
                best_score = s2;
                best = i;
            }
        }
    }
    return best < 0 ? nullptr : node.children[best].get();
}

void add_virtual_loss(PNode &n, int amount) {
    if (amount > 0) n.virtual_loss_count.fetch_add(amount, std::memory_order_relaxed);
}

void remove_virtual_loss(PNode &n, int amount) {
    if (amount <= 0) return;
    const int current = n.virtual_loss_count.fetch_sub(amount, std::memory_order_relaxed);
    if (current < amount) n.virtual_loss_count.store(0, std::memory_order_relaxed);
}

void update(PNode &n, float value) {
    n.visit_count.fetch_add(1, std::memory_order_relaxed);
    float current = n.value_sum.load(std::memory_order_acquire);
    while (!n.value_sum.compare_exchange_weak(current, current + value, std::memory_order_acq_rel,
                                              std::memory_order_acquire)) {
    }
    if (n.virtual_loss_count.load(std::memory_order_relaxed) > 0) {
        const int cur = n.virtual_loss_count.fetch_sub(1, std::memory_order_relaxed);
        if (cur <= 0) n.virtual_loss_count.store(0, std::memory_order_relaxed);
    }
}

}  // namespace

extern "C" {

/* Builds the pointer tree from the arrays of a forest (same meaning as ref_tree's). */
void *ref_ptr_create(int64_t n_nodes, const int32_t *N, const float *W, const float *P, const int32_t *VL,
                     const int32_t *rN, const float *rW, const int32_t *child_begin, const int32_t *child_count,
                     const int32_t *action, const uint32_t *legal) {
    PTree *t = new PTree;
    t->has_rave = rN != nullptr;
    t->nodes.resize((size_t)n_nodes);
    for (int64_t i = 0; i < n_nodes; i++) {
        auto n = std::make_shared<PNode>();
        n->id = (int)i;
        n->action = action ? action[i] : -1;
        n->prior = P[i];
        n->visit_count.store(N[i]);
        n->value_sum.store(W[i]);
        n->virtual_loss_count.store(VL ? VL[i] : 0);
        n->rave_count.store(rN ? rN[i] : 0);
        n->rave_value_sum.store(rW ? rW[i] : 0.0f);
        t->nodes[(size_t)i] = std::move(n);
    }
    for (int64_t i = 0; i < n_nodes; i++) {
        const int cb = child_begin[i], cc = child_count[i];
        if (cc <= 0) continue;
        auto &kids = t->nodes[(size_t)i]->children;
        kids.reserve((size_t)cc);
        for (int j = 0; j < cc; j++) {
            const int64_t id = (int64_t)cb + j;
            if (legal && !((legal[id >> 5] >> (id & 31)) & 1u)) continue;
            kids.push_back(t->nodes[(size_t)id]);
        }
    }
    return t;
}

void ref_ptr_destroy(void *tree) { delete static_cast<PTree *>(tree); }

/* One step: the traversal loop over B traversals (paths[B][max_depth+1], row per traversal,
 * unused entries -1), then the backup loop with the given leaf values; `threads` OpenMP
 * threads.  Returns the seconds spent in the two loops through sel_s / bak_s. */
int ref_ptr_step(void *tree, const int32_t *roots, int32_t B, float c_puct, int32_t virtual_loss, int32_t use_rave,
                 float rave_k, int32_t pw, int32_t max_depth, const float *values, int32_t threads, int32_t *paths,
                 int32_t *path_len, double *sel_s, double *bak_s) {
    PTree *t = static_cast<PTree *>(tree);
    const Params p{c_puct, virtual_loss, use_rave, rave_k, pw, max_depth};
    const int stride = max_depth + 1;
    if (threads < 1) threads = 1;
    const auto t0 = std::chrono::steady_clock::now();
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (int i = 0; i < B; i++) {
        PNode *current = t->nodes[(size_t)roots[i]].get();
        int32_t *row = paths + (size_t)i * stride;
        int len = 0;
        row[len++] = current->id;
        while (!current->children.empty() && len - 1 < max_depth) {
            PNode *child = select_child(*current, p);
            if (!child) break;
            add_virtual_loss(*child, virtual_loss);
            current = child;
            row[len++] = current->id;
        }
        for (int d = len; d < stride; d++) row[d] = -1;
        path_len[i] = len;
    }
    const auto t1 = std::chrono::steady_clock::now();
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (int i = 0; i < B; i++) {
        float v = values[i];
        const int32_t *row = paths + (size_t)i * stride;
        for (int d = path_len[i] - 1; d >= 0; d--) {
            PNode &n = *t->nodes[(size_t)row[d]];
            update(n, v);
            remove_virtual_loss(n, virtual_loss);
            v = -v;
        }
    }
    const auto t2 = std::chrono::steady_clock::now();
    if (sel_s) *sel_s = std::chrono::duration<double>(t1 - t0).count();
    if (bak_s) *bak_s = std::chrono::duration<double>(t2 - t1).count();
    return 0;
}

/* Statistics back into arrays (for the one-thread comparison with ref_cpu). */
void ref_ptr_download(void *tree, int32_t *N, float *W, int32_t *VL) {
    PTree *t = static_cast<PTree *>(tree);
    for (size_t i = 0; i < t->nodes.size(); i++) {
        N[i] = t->nodes[i]->visit_count.load();
        W[i] = t->nodes[i]->value_sum.load();
        VL[i] = t->nodes[i]->virtual_loss_count.load();
    }
}

int64_t ref_ptr_node_bytes(void) { return (int64_t)sizeof(PNode); }

}  // extern "C"
