/*
 * ref_cpu.c -- see ref_cpu.h.  TEST INFRASTRUCTURE ONLY: the checker and the
 * timed CPU baseline, never part of the shipped path.
 *
 * Build: gcc -O2 -std=c11 -ffp-contract=off -fno-fast-math -fPIC -shared
 */
#include "ref_cpu.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

static inline int is_legal(const ref_tree *t, int32_t id) {
    return t->legal == NULL || ((t->legal[(uint32_t)id >> 5] >> ((uint32_t)id & 31u)) & 1u);
}

/* mcts_node.cpp:657-678 -- blend of the Monte-Carlo mean and the RAVE mean.
 * Virtual loss is not part of it. */
float ref_combined_value(const ref_tree *t, int32_t node, float rave_k) {
    int visits = t->N[node];
    int rave_visits = t->rN ? t->rN[node] : 0;
    if (visits == 0 && rave_visits == 0) {
        return 0.0f;
    }
    float mcts_value = visits > 0 ? t->W[node] / (float)visits : 0.0f;
    float rave_value = rave_visits > 0 ? (t->rW ? t->rW[node] : 0.0f) / (float)rave_visits : 0.0f;
    /* "3 * visits + rave_constant": the product is an int, the sum a float */
    int three_v = (int)(3u * (uint32_t)visits);
    float beta = sqrtf(rave_k / ((float)three_v + rave_k));
    float a = (1.0f - beta) * mcts_value;
    float b = beta * rave_value;
    return a + b;
}

/* mcts_node.cpp:143-160 (first loop) and :196-214 (second loop). */
void ref_child_scores(const ref_tree *t, int32_t parent, int32_t child, const ref_params *p,
                      float *score_first, float *score_second) {
    /* mcts_node.cpp:94-95: the parent's raw visit count, no virtual loss */
    float exploration_param = p->c_puct * sqrtf((float)t->N[parent]);

    int child_visits = t->N[child];
    float child_value = t->W[child];
    int virtual_losses = t->VL[child];
    int effective_visits = (int)((uint32_t)child_visits + (uint32_t)virtual_losses);
    float effective_value = child_value - (float)virtual_losses;

    float exploitation = effective_visits > 0 ? effective_value / (float)effective_visits : 0.0f;
    /* first loop divides by the float sum 1.0f + ev */
    float prod = t->P[child] * exploration_param;
    float exploration = prod / (1.0f + (float)effective_visits);
    *score_first = exploitation + exploration;

    /* second loop divides by the int sum 1 + ev, and swaps in the RAVE blend */
    float exploitation2 = p->use_rave ? ref_combined_value(t, child, p->rave_k) : exploitation;
    int one_plus = (int)(1u + (uint32_t)effective_visits);
    float exploration2 = prod / (float)one_plus;
    *score_second = exploitation2 + exploration2;
}

/* smallest k >= 1 with k*k >= n */
int32_t ref_ceil_sqrt(int32_t n) {
    if (n <= 1) return 1;
    int64_t k = (int64_t)sqrt((double)n);
    while (k * k < (int64_t)n) k++;
    while ((k - 1) * (k - 1) >= (int64_t)n) k--;
    return (int32_t)k;
}

/* Progressive-widening eligibility: child takes part iff fewer than k legal siblings
 * beat it by (prior descending, index ascending). */
static void pw_eligible(const ref_tree *t, int32_t cb, int32_t cc, int32_t k, uint8_t *elig) {
    int sorted = 1;
    for (int32_t i = 0; i < cc; i++) {
        if (!is_legal(t, cb + i)) { sorted = 0; break; }
        if (i > 0 && !(t->P[cb + i - 1] >= t->P[cb + i])) { sorted = 0; break; }
    }
    if (sorted) { /* prior-descending storage: the first k children */
        for (int32_t i = 0; i < cc; i++) elig[i] = (uint8_t)(i < k);
        return;
    }
    for (int32_t i = 0; i < cc; i++) {
        if (!is_legal(t, cb + i)) { elig[i] = 0; continue; }
        int32_t rank = 0;
        float pi = t->P[cb + i];
        for (int32_t j = 0; j < cc; j++) {
            if (j == i || !is_legal(t, cb + j)) continue;
            float pj = t->P[cb + j];
            if (pj > pi || (pj == pi && j < i)) rank++;
        }
        elig[i] = (uint8_t)(rank < k);
    }
}

/* mcts_node.cpp:90-236.  The pending-evaluation flags of the reference node are always
 * clear on this path (they are set by evaluator plumbing that is not part of it), so
 * every skip on them is a no-op.  Returns the chosen child's node id, or -1. */
int32_t ref_select_child(const ref_tree *t, int32_t node, const ref_params *p, ref_select_info *info) {
    const int32_t cb = t->child_begin[node];
    const int32_t cc = t->child_count[node];
    float best_score = -INFINITY;
    int32_t best = -1;
    int32_t ncand = 0;

    uint8_t stack_elig[512];
    uint8_t *elig = NULL;
    if (p->pw && cc > 0) {
        elig = cc <= 512 ? stack_elig : (uint8_t *)malloc((size_t)cc);
        pw_eligible(t, cb, cc, ref_ceil_sqrt(t->N[node]), elig);
    }
#define TAKES_PART(i) (is_legal(t, cb + (i)) && (!elig || elig[i]))

    /* first loop: plain PUCT, keep the first strict maximum */
    for (int32_t i = 0; i < cc; i++) {
        if (!TAKES_PART(i)) continue;
        float s1, s2;
        ref_child_scores(t, node, cb + i, p, &s1, &s2);
        if (s1 > best_score) { best_score = s1; best = i; }
        ncand++;
    }
    if (best < 0 && ncand > 0) {
        /* mcts_node.cpp:173-181: no score beat -inf (all NaN or -inf): least visited, first minimum */
        int min_visits = INT32_MAX;
        for (int32_t i = 0; i < cc; i++) {
            if (!TAKES_PART(i)) continue;
            if (t->N[cb + i] < min_visits) { min_visits = t->N[cb + i]; best = i; }
        }
    } else if (best >= 0) {
        /* mcts_node.cpp:184-220: second scan over the same children, best_score carried over */
        for (int32_t i = 0; i < cc; i++) {
            if (!TAKES_PART(i)) continue;
            float s1, s2;
            ref_child_scores(t, node, cb + i, p, &s1, &s2);
            if (s2 > best_score) { best_score = s2; best = i; }
        }
    }

    if (info) {
        /* best candidate of any other child, over both scans */
        float second = -INFINITY;
        for (int32_t i = 0; i < cc; i++) {
            if (i == best || !TAKES_PART(i)) continue;
            float s1, s2;
            ref_child_scores(t, node, cb + i, p, &s1, &s2);
            if (s1 > second) second = s1;
            if (s2 > second) second = s2;
        }
        info->best = best_score;
        info->second = second;
        info->n_candidates = ncand;
        float m = fmaxf(fabsf(best_score), fabsf(second));
        info->near_tie = (best >= 0 && ncand > 1 && isfinite(second) && isfinite(best_score) &&
                          fabsf(best_score - second) <= 1e-6f * m) ? 1 : 0;
    }
#undef TAKES_PART
    if (elig && elig != stack_elig) free(elig);
    return best < 0 ? -1 : cb + best;
}

/* mcts_node_virtual_loss.cpp:15-20 */
void ref_add_vl(ref_tree *t, int32_t node, int32_t amount) {
    if (amount > 0) {
        t->VL[node] = (int32_t)((uint32_t)t->VL[node] + (uint32_t)amount);
    }
}

/* mcts_node_virtual_loss.cpp:22-30 */
void ref_remove_vl1(ref_tree *t, int32_t node) {
    int current = t->VL[node];
    t->VL[node] = (int32_t)((uint32_t)current - 1u);
    if (current <= 0) {
        t->VL[node] = 0;
    }
}

/* mcts_node_virtual_loss.cpp:32-42 */
void ref_remove_vl(ref_tree *t, int32_t node, int32_t amount) {
    if (amount <= 0) return;
    int current = t->VL[node];
    t->VL[node] = (int32_t)((uint32_t)current - (uint32_t)amount);
    if (current < amount) {
        t->VL[node] = 0;
    }
}

/* mcts_node_virtual_loss.cpp:54-71 -- note the trailing removal of one virtual loss */
void ref_update(ref_tree *t, int32_t node, float value) {
    t->N[node] = (int32_t)((uint32_t)t->N[node] + 1u);
    t->W[node] = t->W[node] + value;
    if (t->VL[node] > 0) {
        ref_remove_vl1(t, node);
    }
}

/* mcts_engine_batch_tree_simple.cpp:73-185 run by one thread, traversals in index order:
 * descend while the node is expanded, select, add virtual loss to the selected child
 * (never to the root), record it. */
int ref_select_batch(ref_tree *t, const int32_t *roots, int32_t B, const ref_params *p,
                     int32_t *paths, int32_t *path_len, int32_t *leaf, int32_t *near_tie_depth) {
    const int32_t stride = p->max_depth + 1;
    for (int32_t i = 0; i < B; i++) {
        int32_t *path = paths + (int64_t)i * stride;
        for (int32_t d = 0; d < stride; d++) path[d] = -1;
        int32_t current = roots[i];
        if (current < 0 || current >= t->n_nodes) return -1;
        int32_t len = 0;
        path[len++] = current;
        if (near_tie_depth) near_tie_depth[i] = -1;
        while (t->child_count[current] > 0 && len <= p->max_depth) {
            ref_select_info info;
            int32_t best = ref_select_child(t, current, p, near_tie_depth ? &info : NULL);
            if (best < 0) break;
            if (near_tie_depth && info.near_tie && near_tie_depth[i] < 0) near_tie_depth[i] = len - 1;
            ref_add_vl(t, best, p->virtual_loss);
            current = best;
            path[len++] = current;
        }
        path_len[i] = len;
        leaf[i] = current;
    }
    return 0;
}

void ref_apply_vl_paths(ref_tree *t, const int32_t *paths, const int32_t *path_len, int32_t B,
                        int32_t stride, int32_t amount) {
    for (int32_t i = 0; i < B; i++)
        for (int32_t d = 1; d < path_len[i]; d++) ref_add_vl(t, paths[(int64_t)i * stride + d], amount);
}

void ref_revert_vl_paths(ref_tree *t, const int32_t *paths, const int32_t *path_len, int32_t B,
                         int32_t stride, int32_t amount) {
    for (int32_t i = 0; i < B; i++)
        for (int32_t d = path_len[i] - 1; d >= 0; d--) ref_remove_vl(t, paths[(int64_t)i * stride + d], amount);
}

/* mcts_engine_batch_tree_simple.cpp:276-281, results in index order: leaf to root,
 * update, revert, flip the sign for the opponent. */
void ref_backup_batch(ref_tree *t, const int32_t *paths, const int32_t *path_len,
                      const float *values, int32_t B, int32_t stride, int32_t amount) {
    for (int32_t i = 0; i < B; i++) {
        float value = values[i];
        for (int32_t d = path_len[i] - 1; d >= 0; d--) {
            int32_t node = paths[(int64_t)i * stride + d];
            ref_update(t, node, value);
            ref_remove_vl(t, node, amount);
            value = -value;
        }
    }
}

/* mcts_engine_batch_tree_simple.cpp:114,174-178: the recorded move of every selected child */
void ref_gather_actions(const ref_tree *t, const int32_t *paths, const int32_t *path_len,
                        int32_t B, int32_t stride, int32_t *actions) {
    const int32_t astride = stride - 1;
    for (int32_t i = 0; i < B; i++) {
        for (int32_t d = 0; d < astride; d++) {
            int32_t v = -1;
            if (d + 1 < path_len[i]) {
                int32_t node = paths[(int64_t)i * stride + d + 1];
                v = t->action ? t->action[node] : node;
            }
            actions[(int64_t)i * astride + d] = v;
        }
    }
}

/* ---- open-addressing transposition table ---- */

#define REF_TT_EMPTY (~(uint64_t)0)

static inline uint64_t tt_home(uint64_t key, int32_t log2_slots) {
    return (key * 0x9E3779B97F4A7C15ull) >> (64 - log2_slots);
}

void ref_tt_clear(ref_tt_slot *slots, int32_t log2_slots) {
    uint64_t n = (uint64_t)1 << log2_slots;
    for (uint64_t i = 0; i < n; i++) {
        slots[i].key = REF_TT_EMPTY;
        slots[i].node = -1;
        slots[i].depth = 0;
    }
}

int ref_tt_insert(ref_tt_slot *slots, int32_t log2_slots, uint64_t key, int32_t node, int32_t depth) {
    if (key == REF_TT_EMPTY) return -2;
    uint64_t mask = ((uint64_t)1 << log2_slots) - 1;
    uint64_t s = tt_home(key, log2_slots);
    for (uint64_t probe = 0; probe <= mask; probe++, s = (s + 1) & mask) {
        if (slots[s].key == key) return 1;
        if (slots[s].key == REF_TT_EMPTY) {
            slots[s].key = key;
            slots[s].node = node;
            slots[s].depth = depth;
            return 0;
        }
    }
    return -1;
}

int64_t ref_tt_probe(const ref_tt_slot *slots, int32_t log2_slots, const uint64_t *keys, int64_t n,
                     int32_t min_depth, int32_t *out_node) {
    uint64_t mask = ((uint64_t)1 << log2_slots) - 1;
    int64_t hits = 0;
    for (int64_t i = 0; i < n; i++) {
        uint64_t key = keys[i];
        int32_t found = -1;
        if (key != REF_TT_EMPTY) {
            uint64_t s = tt_home(key, log2_slots);
            for (uint64_t probe = 0; probe <= mask; probe++, s = (s + 1) & mask) {
                if (slots[s].key == key) {
                    if (slots[s].depth >= min_depth) found = slots[s].node;
                    break;
                }
                if (slots[s].key == REF_TT_EMPTY) break;
            }
        }
        out_node[i] = found;
        if (found >= 0) hits++;
    }
    return hits;
}

/* ---- PHMapTranspositionTable::store with its replacement policy
 * (src/mcts/phmap_transposition_table.cpp:51-84, createEntry :202-216, Entry::getReplacementScore
 * include/mcts/phmap_transposition_table.h:68-72), over the open-addressing table, entries of a call
 * in index order.  The reference's clock (access_counter_) is shared by its threads and only ticks on
 * some paths; here entry i of a call has the time t0 + i.  Among the entries of one call that carry
 * the same key only the first is stored (see ref_cpu.h).  counts: new entries, replacements,
 * duplicates dropped, -.  Returns 0, -1 when the table is full, -2 on a key equal to the empty marker. */
static float tt_score(uint32_t visits, float value, int32_t depth, uint32_t now, uint32_t last_access) {
    float recency = 1.0f / (1.0f + (float)(now - last_access));
    float importance = (float)visits * (1.0f + value) * (1.0f + (float)depth);
    return recency * importance;
}

int ref_tt_store_batch(ref_tt_slot *slots, ref_tt_meta *meta, int32_t log2_slots, const ref_tree *t,
                       const uint64_t *keys, const int32_t *nodes, const int32_t *depths, int64_t n, uint32_t t0,
                       float threshold, int32_t *counts) {
    uint64_t mask = ((uint64_t)1 << log2_slots) - 1;
    int rc = 0;
    int64_t *touched = (int64_t *)malloc((size_t)(n > 0 ? n : 1) * sizeof(int64_t));
    int64_t n_touched = 0;
    counts[0] = counts[1] = counts[2] = counts[3] = 0;
    for (int64_t i = 0; i < n; i++) {
        if (nodes[i] < 0) continue;                               /* store(): if (!node) return */
        if (keys[i] == REF_TT_EMPTY) { rc = -2; continue; }
        uint64_t s = tt_home(keys[i], log2_slots);
        int placed = 0;
        for (uint64_t probe = 0; probe <= mask && !placed; probe++, s = (s + 1) & mask) {
            if (slots[s].key != keys[i] && slots[s].key != REF_TT_EMPTY) continue;
            placed = 1;
            const int fresh = slots[s].key == REF_TT_EMPTY;
            if (!fresh && meta[s].reserved == 1) { counts[2]++; break; }   /* an earlier entry of this call */
            const int32_t node = nodes[i];
            const int32_t depth = (int32_t)(uint16_t)(depths ? depths[i] : 0);  /* Entry::depth is uint16_t */
            uint32_t visits = 0;
            float value = 0.0f;
            if (node < t->n_nodes) {                              /* createEntry :212-213, getValue :484-490 */
                visits = (uint32_t)t->N[node];
                value = t->N[node] == 0 ? 0.0f : t->W[node] / (float)t->N[node];
            }
            int write = fresh;
            if (fresh) {
                counts[0]++;
            } else {
                const uint32_t now = t0 + (uint32_t)i;            /* :65 */
                const float existing = tt_score(meta[s].visits, meta[s].value, slots[s].depth, now, meta[s].last_access);
                const float incoming = tt_score(visits, value, depth, now, 0u);
                if (incoming > existing * (1.0f + threshold)) { write = 1; counts[1]++; }   /* :71 */
            }
            if (write) {
                slots[s].key = keys[i];
                slots[s].node = node;
                slots[s].depth = depth;
                meta[s].visits = visits;
                meta[s].value = value;
                meta[s].last_access = 0;                          /* a new Entry starts at 0 */
            }
            meta[s].reserved = 1;
            touched[n_touched++] = (int64_t)s;
        }
        if (!placed) rc = rc ? rc : -1;
    }
    for (int64_t j = 0; j < n_touched; j++) meta[touched[j]].reserved = 0;
    free(touched);
    return rc;
}

/* PHMapTranspositionTable::lookup (:86-117) for a batch: a hit that passes the depth test stamps the
 * entry with its time (:107), lookup i at t0 + i.  Returns the number of hits. */
int64_t ref_tt_lookup_batch(const ref_tt_slot *slots, ref_tt_meta *meta, int32_t log2_slots, const uint64_t *keys,
                            int64_t n, int32_t min_depth, uint32_t t0, int32_t *out_node) {
    uint64_t mask = ((uint64_t)1 << log2_slots) - 1;
    int64_t hits = 0;
    for (int64_t i = 0; i < n; i++) {
        int32_t found = -1;
        if (keys[i] != REF_TT_EMPTY) {
            uint64_t s = tt_home(keys[i], log2_slots);
            for (uint64_t probe = 0; probe <= mask; probe++, s = (s + 1) & mask) {
                if (slots[s].key == keys[i]) {
                    if (slots[s].depth >= min_depth) {
                        found = slots[s].node;
                        meta[s].last_access = t0 + (uint32_t)i;
                    }
                    break;
                }
                if (slots[s].key == REF_TT_EMPTY) break;
            }
        }
        out_node[i] = found;
        if (found >= 0) hits++;
    }
    return hits;
}

/* ---- the traversal loop with the transposition table switched on, redirects included
 * (mcts_engine_batch_tree_simple.cpp:88-165; store :116-128, lookup :131-141, redirect :142-156;
 * MCTSNode::updateChildReference mcts_node.cpp:617-630), one thread, traversals in index order.
 *
 * The children vector of a node is the slot range [child_begin, child_begin + child_count); slot s
 * holds node s until updateChildReference re-points it: alias[s] = the node it holds now, -1 = its own.
 * The statistics, the prior and the ACTION the loop reads are those of the node a slot holds
 * (children_[i]->getAction(), :112), so the move recorded for a re-pointed slot is the action of the
 * node it now holds, as in the reference.  The key of a step is getHash() of the root state with the
 * recorded moves replayed (:119-124, :133-137): here node_key of the node of the ORIGINAL tree (slots,
 * not what they hold) that the recorded moves lead to from the root; where that node does not exist
 * (a move no child slot carries, or a node that is not expanded) the position has no key from there on:
 * nothing is stored or looked up (the reference would ask the game).
 * Time: the reference's access counter on one thread, starting at t0: it ticks on a store that finds its key
 * (phmap_transposition_table.cpp:65) and on a lookup that hits (:107), and not otherwise.
 * counts: [0] new entries, [1] replacements, [2] lookups that found an entry, [3] redirects, [4] steps,
 * [5] ticks of the counter.  Returns 0, -1 bad root, -2 table full. */
static int32_t select_slot_redirected(const ref_tree *t, const int32_t *alias, int32_t node, const ref_params *p) {
    const int32_t cb = t->child_begin[node];
    const int32_t cc = t->child_count[node];
    float best_score = -INFINITY;
    int32_t best = -1;
    int32_t ncand = 0;
#define HELD(i) (alias[cb + (i)] >= 0 ? alias[cb + (i)] : cb + (i))
    for (int32_t i = 0; i < cc; i++) {
        if (!is_legal(t, cb + i)) continue;
        float s1, s2;
        ref_child_scores(t, node, HELD(i), p, &s1, &s2);
        if (s1 > best_score) { best_score = s1; best = i; }
        ncand++;
    }
    if (best < 0 && ncand > 0) {
        int min_visits = INT32_MAX;
        for (int32_t i = 0; i < cc; i++) {
            if (!is_legal(t, cb + i)) continue;
            if (t->N[HELD(i)] < min_visits) { min_visits = t->N[HELD(i)]; best = i; }
        }
    } else if (best >= 0) {
        for (int32_t i = 0; i < cc; i++) {
            if (!is_legal(t, cb + i)) continue;
            float s1, s2;
            ref_child_scores(t, node, HELD(i), p, &s1, &s2);
            if (s2 > best_score) { best_score = s2; best = i; }
        }
    }
#undef HELD
    return best < 0 ? -1 : cb + best;
}

int ref_select_redirect_batch(ref_tree *t, int32_t *alias, const int32_t *roots, int32_t B, const ref_params *p,
                              ref_tt_slot *slots, ref_tt_meta *meta, int32_t log2_slots, uint32_t t0, float threshold,
                              const uint64_t *node_key, int32_t *paths, int32_t *path_len, int32_t *leaf,
                              int32_t *moves, int32_t *counts) {
    const int32_t stride = p->max_depth + 1;
    int rc = 0;
    uint32_t g = 0;
    uint32_t clock = t0;  /* access_counter_: ticks on a store that finds its key (:65) and on a lookup that hits (:107) */
    for (int j = 0; j < 6; j++) counts[j] = 0;
    for (int32_t i = 0; i < B; i++) {
        int32_t *path = paths + (int64_t)i * stride;
        int32_t *mv = moves ? moves + (int64_t)i * p->max_depth : NULL;
        for (int32_t d = 0; d < stride; d++) path[d] = -1;
        for (int32_t d = 0; mv && d < p->max_depth; d++) mv[d] = -1;
        int32_t current = roots[i];
        if (current < 0 || current >= t->n_nodes) return -1;
        int32_t shadow = current;  /* node of the original tree the recorded moves lead to */
        int32_t len = 0;
        path[len++] = current;
        while (t->child_count[current] > 0 && len <= p->max_depth) {
            const int32_t slot = select_slot_redirected(t, alias, current, p);
            if (slot < 0) break;
            int32_t best = alias[slot] >= 0 ? alias[slot] : slot;
            ref_add_vl(t, best, p->virtual_loss);                                     /* :109 */
            const int32_t move = t->action ? t->action[best] : best;                 /* :112 */
            if (mv) mv[len - 1] = move;
            if (shadow >= 0) {
                int32_t next = -1;
                for (int32_t c = 0; c < t->child_count[shadow] && next < 0; c++) {
                    const int32_t s = t->child_begin[shadow] + c;
                    if (is_legal(t, s) && (t->action ? t->action[s] : s) == move) next = s;
                }
                shadow = next;
            }
            const uint64_t key = shadow >= 0 ? node_key[shadow] : REF_TT_EMPTY;
            if (key != REF_TT_EMPTY) {
                if (t->N[best] == 0) {                                               /* :116-128 */
                    int32_t c4[4];
                    const int32_t depth = len;                                       /* move_sequence.size() */
                    int r = ref_tt_store_batch(slots, meta, log2_slots, t, &key, &best, &depth, 1, clock, threshold, c4);
                    if (r == -1) rc = -2;
                    else if (c4[0] == 0) clock++;                                    /* the key was there: :65 */
                    counts[0] += c4[0];
                    counts[1] += c4[1];
                }
                int32_t found = -1;
                ref_tt_lookup_batch(slots, meta, log2_slots, &key, 1, 0, clock, &found);         /* :141 */
                if (found >= 0) {
                    counts[2]++;
                    clock++;                                                         /* :107 */
                }
                if (found >= 0 && found != best && found < t->n_nodes && t->N[found] > 0) {  /* :142 */
                    ref_remove_vl(t, best, p->virtual_loss);                         /* :146 */
                    /* :149, updateChildReference: the first slot of `current` that holds the old child */
                    for (int32_t c = 0; c < t->child_count[current]; c++) {
                        const int32_t s = t->child_begin[current] + c;
                        if (is_legal(t, s) && (alias[s] >= 0 ? alias[s] : s) == best) {
                            alias[s] = found;
                            break;
                        }
                    }
                    ref_add_vl(t, found, p->virtual_loss);                           /* :152 */
                    best = found;
                    counts[3]++;
                }
            }
            g++;
            current = best;
            path[len++] = current;
        }
        path_len[i] = len;
        leaf[i] = current;
    }
    counts[4] = (int32_t)g;
    counts[5] = (int32_t)(clock - t0);
    return rc;
}

/* ---- leaf expansion (mcts_node.cpp:238-436, :512-593; call site
 * mcts_engine_batch_tree_simple.cpp:249-259) ---- */
/* mcts_node.cpp:296-341: the number of children expand() creates.  The "incremental expansion"
 * branch (:312-337) needs a node that is already expanded, and such a call has returned at the
 * compare-exchange of :264 before it gets there: what remains is the first expansion. */
int32_t ref_widened_children(int32_t legal, int32_t visits, int32_t use_pw, float cpw, float kpw) {
    size_t num = (size_t)legal;                                   /* :294 */
    if (use_pw) {
        /* :305-308; std::pow(int, float) and its product with a float are double arithmetic */
        double grown = (double)cpw * pow((double)(visits + 1), (double)kpw);
        float as_float = (float)grown;
        float at_least = as_float > 8.0f ? as_float : 8.0f;       /* std::max(8.0f, x): 8.0f when x is NaN */
        size_t target = at_least >= 1.0e18f ? (size_t)legal : (size_t)at_least;
        if (target > (size_t)legal) target = (size_t)legal;      /* std::min(legal_moves.size(), ...) */
        num = target > 1 ? target : 1;                            /* :340 */
    }
    if (num > (size_t)legal) num = (size_t)legal;                 /* the loop stops at legal_moves.size(), :367 */
    return (int32_t)num;
}

int64_t ref_expand_batch_ex(int64_t n_nodes, int64_t capacity, int32_t *N, float *W, float *P, int32_t *VL,
                            int32_t *rN, float *rW, int32_t *child_begin, int32_t *child_count, int32_t *action,
                            uint32_t *legal, const int32_t *leaf, int32_t B, const int32_t *move_begin,
                            const int32_t *moves, const int32_t *policy_begin, const float *policy,
                            int32_t action_space, int32_t use_pw, float cpw, float kpw, int32_t *first_child) {
    /* first pass: how many nodes would be added (a leaf counts once: child_count is set below,
     * so a dry run has to remember the leaves it has seen) */
    int64_t need = 0;
    for (int32_t t = 0; t < B; t++) {
        int32_t cnt = move_begin[t + 1] - move_begin[t];
        if (cnt <= 0 || leaf[t] < 0 || child_count[leaf[t]] != 0) continue;
        int seen = 0;
        for (int32_t u = 0; u < t && !seen; u++)
            seen = leaf[u] == leaf[t] && move_begin[u + 1] - move_begin[u] > 0;
        if (seen) continue;
        if (cnt > 1000) cnt = 1000;
        need += ref_widened_children(cnt, N[leaf[t]], use_pw, cpw, kpw);
    }
    if (n_nodes + need > capacity) return -1;
    for (int32_t t = 0; t < B; t++) {
        if (first_child) first_child[t] = -1;
        int32_t cnt = move_begin[t + 1] - move_begin[t];
        if (cnt <= 0 || leaf[t] < 0) continue;         /* terminal: stays a leaf */
        int32_t node = leaf[t];
        if (child_count[node] != 0) continue;           /* already expanded: first caller won */
        if (cnt > 1000) cnt = 1000;                     /* max_reasonable_moves */
        cnt = ref_widened_children(cnt, N[node], use_pw, cpw, kpw);
        /* setPriorProbabilities is only called with a policy that is not empty
         * (mcts_engine_batch_tree_simple.cpp:256-258) */
        const int32_t psize = policy_begin ? policy_begin[t + 1] - policy_begin[t] : 0;
        const float *pol = psize > 0 ? policy + policy_begin[t] : NULL;
        const int32_t begin = (int32_t)n_nodes;
        for (int32_t i = 0; i < cnt; i++) {
            const int32_t id = begin + i;
            const int32_t mv = moves[move_begin[t] + i];
            float prior;
            if (!pol) {
                prior = 1.0f / (float)cnt;              /* expand(): uniform_prior, :426-429 */
            } else if (psize == action_space) {         /* :537-560 */
                if (mv >= 0 && mv < action_space) {
                    prior = pol[mv];
                    prior = prior > 0.0f ? prior : 0.0f;    /* std::min(1.0f, std::max(0.0f, prob)) */
                    prior = prior < 1.0f ? prior : 1.0f;
                } else {
                    prior = 0.01f;                      /* action out of bounds */
                }
            } else if (psize == cnt) {                  /* :561-575: by child index */
                prior = pol[i];
                prior = prior > 0.0f ? prior : 0.0f;
                prior = prior < 1.0f ? prior : 1.0f;
            } else {
                prior = 1.0f / (float)cnt;              /* :576-584: size mismatch, uniform */
            }
            N[id] = 0;
            W[id] = 0.0f;
            P[id] = prior;
            VL[id] = 0;
            if (rN) rN[id] = 0;
            if (rW) rW[id] = 0.0f;
            child_begin[id] = 0;
            child_count[id] = 0;
            if (action) action[id] = mv;
            if (legal) legal[(uint32_t)id >> 5] |= 1u << ((uint32_t)id & 31u);
        }
        child_begin[node] = begin;
        child_count[node] = cnt;
        n_nodes += cnt;
        if (first_child) first_child[t] = begin;
    }
    return n_nodes;
}

/* The common case: one policy row of action_space values per traversal (or none), no widening. */
int64_t ref_expand_batch(int64_t n_nodes, int64_t capacity, int32_t *N, float *W, float *P, int32_t *VL,
                         int32_t *rN, float *rW, int32_t *child_begin, int32_t *child_count, int32_t *action,
                         uint32_t *legal, const int32_t *leaf, int32_t B, const int32_t *move_begin,
                         const int32_t *moves, const float *policy, int32_t action_space, int32_t *first_child) {
    int32_t *pb = NULL;
    if (policy) {
        pb = (int32_t *)malloc(((size_t)B + 1) * sizeof(int32_t));
        for (int32_t t = 0; t <= B; t++) pb[t] = t * action_space;
    }
    int64_t r = ref_expand_batch_ex(n_nodes, capacity, N, W, P, VL, rN, rW, child_begin, child_count, action, legal,
                                    leaf, B, move_begin, moves, pb, policy, action_space, 0, 0.0f, 0.0f, first_child);
    free(pb);
    return r;
}

/* ---- MCTSEngine::getActionProbabilities (src/mcts/mcts_engine_tree.cpp:388-465) ---- */
/* src/mcts/mcts_engine_eval.cpp:78-110 (MCTSEngine::addDirichletNoise) from the samples on:
 * gamma[] holds one gamma(alpha, 1) draw per child of root, in child order (the reference
 * draws them from std::gamma_distribution on its engine, :83-90).  Returns the number of
 * children, or -1 when n_gamma does not match it. */
int32_t ref_add_root_noise(ref_tree *t, int32_t root, const float *gamma, int32_t n_gamma, float epsilon) {
    const int32_t cb = t->child_begin[root], cc = t->child_count[root];
    int32_t children = 0;
    for (int32_t i = 0; i < cc; i++) children += is_legal(t, cb + i) ? 1 : 0;
    if (children == 0) return 0; /* :78-80 */
    if (n_gamma != children) return -1;
    float sum = 0.0f; /* std::accumulate(..., 0.0f): left to right */
    for (int32_t j = 0; j < children; j++) sum = sum + gamma[j];
    int32_t j = 0;
    for (int32_t i = 0; i < cc; i++) {
        if (!is_legal(t, cb + i)) continue;
        float n = sum > 0.0f ? gamma[j] / sum : 1.0f / (float)children; /* :93-101 */
        float keep = (1.0f - epsilon) * t->P[cb + i];
        float add = epsilon * n;
        t->P[cb + i] = keep + add; /* :104-110 */
        j++;
    }
    return children;
}

int32_t ref_action_probabilities(const ref_tree *t, int32_t root, float temperature, int32_t action_space,
                                 float *out) {
    for (int32_t a = 0; a < action_space; a++) out[a] = 0.0f;
    const int32_t cb = t->child_begin[root], cc = t->child_count[root];
    /* the children: slots of the range whose legal bit is set */
    int32_t n = 0;
    for (int32_t i = 0; i < cc; i++) {
        const int32_t id = cb + i;
        if (t->legal && !((t->legal[(uint32_t)id >> 5] >> ((uint32_t)id & 31u)) & 1u)) continue;
        n++;
    }
    if (n == 0) return 0;
    float max_count = 0.0f;
    int32_t max_idx = -1;
    for (int32_t i = 0; i < cc; i++) {
        const int32_t id = cb + i;
        if (t->legal && !((t->legal[(uint32_t)id >> 5] >> ((uint32_t)id & 31u)) & 1u)) continue;
        const float c = (float)t->N[id];
        if (max_idx < 0 || c > max_count) { /* std::max_element: first of the largest */
            max_count = c;
            max_idx = id;
        }
    }
    float sum = 0.0f;
    const int near_zero = temperature < 0.01f;
    if (!near_zero && max_count > 0.0f) {
        for (int32_t i = 0; i < cc; i++) {
            const int32_t id = cb + i;
            if (t->legal && !((t->legal[(uint32_t)id >> 5] >> ((uint32_t)id & 31u)) & 1u)) continue;
            const float c = (float)t->N[id];
            float scaled = 0.0f;
            if (c > 0.0f) scaled = powf(c / max_count, 1.0f / temperature);
            sum += scaled;
        }
    }
    for (int32_t i = 0; i < cc; i++) {
        const int32_t id = cb + i;
        if (t->legal && !((t->legal[(uint32_t)id >> 5] >> ((uint32_t)id & 31u)) & 1u)) continue;
        float prob;
        if (near_zero) {
            prob = id == max_idx ? 1.0f : 0.0f;
        } else if (max_count <= 0.0f || !(sum > 0.0f)) {
            prob = 1.0f / (float)n; /* 1.0f / counts.size() */
        } else {
            const float c = (float)t->N[id];
            float scaled = 0.0f;
            if (c > 0.0f) scaled = powf(c / max_count, 1.0f / temperature);
            prob = scaled / sum;
        }
        const int32_t a = t->action ? t->action[id] : id;
        if (a >= 0 && a < action_space) out[a] = prob;
    }
    return n;
}

/* ---- tree reuse (src/mcts/mcts_engine_search.cpp:1029-1075) ---- */
int32_t ref_reroot_child(const ref_tree *t, int32_t root, int32_t last_action) {
    if (last_action < 0) return -1; /* :1039 */
    const int32_t cb = t->child_begin[root], cc = t->child_count[root];
    for (int32_t i = 0; i < cc; i++) {
        const int32_t id = cb + i;
        if (t->legal && !((t->legal[(uint32_t)id >> 5] >> ((uint32_t)id & 31u)) & 1u)) continue;
        const int32_t a = t->action ? t->action[id] : id;
        if (a == last_action) return id;
    }
    return -1;
}

int64_t ref_compact_order(const ref_tree *t, int32_t new_root, int32_t *old_of_new) {
    int64_t head = 0, tail = 0;
    old_of_new[tail++] = new_root;
    while (head < tail) {
        const int32_t old = old_of_new[head++];
        const int32_t cb = t->child_begin[old], cc = t->child_count[old];
        for (int32_t i = 0; i < cc; i++) old_of_new[tail++] = cb + i; /* empty slots keep their place */
    }
    return tail;
}

/* ---- RAVE statistics of backPropagate (src/mcts/mcts_engine_tree.cpp:288-331) ---- */
void ref_rave_backup_batch(ref_tree *t, const int32_t *paths, const int32_t *path_len, const float *values,
                           int32_t B, int32_t stride) {
    if (!t->rN || !t->rW) return;
    for (int32_t i = 0; i < B; i++) {
        const int32_t *path = paths + (int64_t)i * stride;
        const int32_t len = path_len[i];
        int invert = 0;
        for (int32_t d = len - 1; d >= 0; d--) { /* leaf to root */
            const int32_t node = path[d];
            const float v = invert ? -values[i] : values[i];
            const int32_t cb = t->child_begin[node], cc = t->child_count[node];
            for (int32_t c = 0; c < cc; c++) {
                const int32_t id = cb + c;
                if (t->legal && !((t->legal[(uint32_t)id >> 5] >> ((uint32_t)id & 31u)) & 1u)) continue;
                const int32_t a = t->action ? t->action[id] : id;
                for (int32_t e = 0; e < len; e++) {
                    const int32_t pa = t->action ? t->action[path[e]] : path[e];
                    if (pa != -1 && pa == a) {
                        t->rN[id] += 1;
                        t->rW[id] += v;
                        break; /* once per child */
                    }
                }
            }
            invert = !invert;
        }
    }
}

/* ---- position keys (src/utils/zobrist_hash.cpp:9-36,129-131; src/games/gomoku/gomoku_state.cpp:947-957) ---- */

/* std::mt19937_64, the generator ZobristHash draws from (zobrist_hash.cpp:20): the published
 * MT19937-64 recurrence (n = 312, m = 156, r = 31, a = 0xB5026F5AA96619E9, tempering
 * 29/0x5555555555555555, 17/0x71D67FFFEDA60000, 37/0xFFF7EEE000000000, 43) and the seeding
 * x_i = 6364136223846793005 * (x_{i-1} ^ (x_{i-1} >> 62)) + i of the C++ standard. */
void ref_mt64_seed(ref_mt64 *g, uint64_t seed) {
    g->mt[0] = seed;
    for (int i = 1; i < 312; i++) g->mt[i] = 6364136223846793005ull * (g->mt[i - 1] ^ (g->mt[i - 1] >> 62)) + (uint64_t)i;
    g->idx = 312;
}

uint64_t ref_mt64_next(ref_mt64 *g) {
    if (g->idx >= 312) {
        for (int i = 0; i < 312; i++) {
            const uint64_t x = (g->mt[i] & 0xFFFFFFFF80000000ull) | (g->mt[(i + 1) % 312] & 0x7FFFFFFFull);
            g->mt[i] = g->mt[(i + 156) % 312] ^ (x >> 1) ^ ((x & 1ull) ? 0xB5026F5AA96619E9ull : 0ull);
        }
        g->idx = 0;
    }
    uint64_t y = g->mt[g->idx++];
    y ^= (y >> 29) & 0x5555555555555555ull;
    y ^= (y << 17) & 0x71D67FFFEDA60000ull;
    y ^= (y << 37) & 0xFFF7EEE000000000ull;
    y ^= y >> 43;
    return y;
}

/* ZobristHash::ZobristHash(boardSize, numPieceTypes, numPlayers, seed), zobrist_hash.cpp:9-36: one
 * generator seeded with `seed` (an unsigned: 32 bits), piece tables first (piece-major,
 * boardSize * boardSize keys each), then the player keys.  seed 0 means "from the clock" there
 * and is refused here. */
int ref_zobrist_tables(int32_t board_size, int32_t n_piece, int32_t n_players, uint32_t seed, uint64_t *piece,
                       uint64_t *player) {
    if (board_size <= 0 || n_piece < 0 || n_players <= 0 || seed == 0) return -1;
    ref_mt64 g;
    ref_mt64_seed(&g, (uint64_t)seed);
    const int64_t per = (int64_t)board_size * board_size;
    for (int32_t p = 0; p < n_piece; p++)
        for (int64_t pos = 0; pos < per; pos++) piece[(int64_t)p * per + pos] = ref_mt64_next(&g);
    for (int32_t p = 0; p < n_players; p++) player[p] = ref_mt64_next(&g);
    return 0;
}

/* GomokuState::compute_hash_signature_internal, gomoku_state.cpp:947-957: for both sides, for every
 * cell in ascending order, a stone of that side folds in getPieceHash(side, cell); then
 * getPlayerHash(current_player - 1).  board[cell] = 0 empty, 1 BLACK, 2 WHITE. */
uint64_t ref_position_key(const int8_t *board, int32_t cells, const uint64_t *piece, int64_t piece_stride,
                          const uint64_t *player, int32_t current_player) {
    uint64_t h = 0;
    for (int32_t p_idx = 0; p_idx < 2; p_idx++)
        for (int32_t action = 0; action < cells; action++)
            if (board[action] == p_idx + 1) h ^= piece[(int64_t)p_idx * piece_stride + action];
    h ^= player[current_player - 1];
    return h;
}

/* The temp_state of the traversal loop (mcts_engine_batch_tree_simple.cpp:119-124,133-137): a
 * clone of the root state, makeMove for every move of the path (make_move_internal,
 * gomoku_state.cpp:963-980: the side to move places a stone, then the other side is to move),
 * getHash() computed from the resulting board.  Returns the number of paths with a move that is
 * off the board or on an occupied cell (their key is ~0). */
int32_t ref_leaf_keys(const ref_tree *t, const int32_t *paths, const int32_t *path_len, int32_t B, int32_t stride,
                      const int8_t *root_boards, const int32_t *root_player, int32_t cells, const uint64_t *piece,
                      int64_t piece_stride, const uint64_t *player, uint64_t *out) {
    int32_t bad = 0;
    int8_t *board = (int8_t *)malloc((size_t)cells);
    for (int32_t i = 0; i < B; i++) {
        memcpy(board, root_boards + (int64_t)i * cells, (size_t)cells);
        int32_t cur = root_player[i];
        int ok = path_len[i] >= 1;
        for (int32_t d = 1; ok && d < path_len[i]; d++) {
            const int32_t node = paths[(int64_t)i * stride + d];
            const int32_t a = t->action ? t->action[node] : node;
            if (a < 0 || a >= cells || board[a] != 0) {
                ok = 0;
                break;
            }
            board[a] = (int8_t)cur;
            cur = cur == 1 ? 2 : 1;
        }
        out[i] = ok ? ref_position_key(board, cells, piece, piece_stride, player, cur) : ~0ull;
        bad += !ok;
    }
    free(board);
    return bad;
}
