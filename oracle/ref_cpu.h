/*
 * ref_cpu -- CPU restatement of the reference's tree-search arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This is the checker the HIP path is compared
 * against and the timed CPU baseline.  Nothing in the shipped library may
 * call, link or load it; only tests, the smoke check and the benchmark's
 * cpu_baseline leg do.
 *
 * Every function restates one piece of the reference (paths relative to the
 * reference checkout):
 *   ref_select_child      src/mcts/mcts_node.cpp:90-236   (MCTSNode::selectChild)
 *   ref_combined_value    src/mcts/mcts_node.cpp:657-678  (MCTSNode::getCombinedValue)
 *   ref_add_vl            src/mcts/mcts_node_virtual_loss.cpp:15-20
 *   ref_remove_vl1        src/mcts/mcts_node_virtual_loss.cpp:22-30
 *   ref_remove_vl         src/mcts/mcts_node_virtual_loss.cpp:32-42
 *   ref_update            src/mcts/mcts_node_virtual_loss.cpp:54-71
 *   ref_select_batch      src/mcts/mcts_engine_batch_tree_simple.cpp:73-185 (one thread, i ascending)
 *   ref_backup_batch      src/mcts/mcts_engine_batch_tree_simple.cpp:242-282 (i ascending)
 *   ref_expand_batch      src/mcts/mcts_node.cpp:238-436, :512-593 (MCTSNode::expand, setPriorProbabilities),
 *                         call site src/mcts/mcts_engine_batch_tree_simple.cpp:249-259
 *   ref_action_probabilities  src/mcts/mcts_engine_tree.cpp:388-465 (MCTSEngine::getActionProbabilities)
 *   ref_add_root_noise    src/mcts/mcts_engine_eval.cpp:78-110 (MCTSEngine::addDirichletNoise, from the
 *                         gamma samples on)
 *   ref_rave_backup_batch src/mcts/mcts_engine_tree.cpp:288-331 (RAVE part of backPropagate; not dispatched
 *                         by the reference's live search loop)
 *   ref_reroot_child      src/mcts/mcts_engine_search.cpp:1029-1075 (searchWithTreeReuse)
 *   ref_mt64_*, ref_zobrist_tables  src/utils/zobrist_hash.cpp:9-36,129-131 (std::mt19937_64 stream of the tables)
 *   ref_position_key      src/games/gomoku/gomoku_state.cpp:947-957 (compute_hash_signature_internal)
 *   ref_leaf_keys         src/mcts/mcts_engine_batch_tree_simple.cpp:119-124,133-137 (clone, replay, getHash)
 *   ref_tt_*              call sites src/mcts/mcts_engine_batch_tree_simple.cpp:126,141 and
 *                         src/mcts/phmap_transposition_table.cpp:51-117
 *   ref_select_redirect_batch  src/mcts/mcts_engine_batch_tree_simple.cpp:88-165 with the table on
 *                         (redirect :142-156, MCTSNode::updateChildReference src/mcts/mcts_node.cpp:617-630)
 *
 * The node record of include/mcts/mcts_node.h:160-178 is flattened into
 * arrays indexed by node id; the children of a node are the contiguous id
 * range [child_begin, child_begin + child_count).
 *
 * Pinned by: the reference's own unit-test facts (tests/mcts/mcts_node_test.cpp:237-313,
 * tests/mcts/virtual_loss_test.cpp:42-69,160-224,282-308), the recorded known-answer
 * table of the compiled reference node class (tests/golden/kat_reference.json), closed
 * forms and a double-precision brute force (tests/test_oracle_*.py).
 *
 * PARITY UNPINNED (no reference behaviour exists to pin them; defined here):
 *   - the progressive-widening eligibility filter (pw != 0): top ceil(sqrt(N_parent))
 *     children by prior, ties to the lower child index;
 *   - the open-addressing transposition table (the reference delegates to the
 *     absent third-party parallel-hashmap v1.3.8); checked against a brute-force map;
 *   - the ORDER of the children that leaf expansion creates (the reference shuffles the
 *     legal moves with a random seed; the order offered is kept here).  The rest of
 *     expansion is pinned by tests/test_oracle_expand.py.
 *
 * Must be compiled with -ffp-contract=off and without -ffast-math: the reference
 * translation unit is built for baseline x86-64 (no FMA), IEEE binary32, round to nearest.
 */
#ifndef OMK_ORACLE_REF_CPU_H
#define OMK_ORACLE_REF_CPU_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ref_tree {
    int64_t n_nodes;
    int32_t *N;                 /* visit_count_            */
    float *W;                   /* value_sum_              */
    float *P;                   /* prior_probability_      */
    int32_t *VL;                /* virtual_loss_count_     */
    int32_t *rN;                /* rave_count_     (NULL = all zero) */
    float *rW;                  /* rave_value_sum_ (NULL = all zero) */
    const int32_t *child_begin; /* first child id          */
    const int32_t *child_count; /* 0 = not expanded (isLeaf) */
    const int32_t *action;      /* action_ (may be NULL)   */
    const uint32_t *legal;      /* bit per node id, 1 = the slot holds a child; NULL = all */
} ref_tree;

typedef struct ref_params {
    float c_puct;         /* MCTSSettings::exploration_constant */
    int32_t virtual_loss; /* MCTSSettings::virtual_loss         */
    int32_t use_rave;     /* MCTSSettings::use_rave             */
    float rave_k;         /* MCTSSettings::rave_constant        */
    int32_t pw;           /* selection-time progressive widening (0 = off) */
    int32_t max_depth;    /* bound on selection steps per traversal (buffer size; the reference has none) */
} ref_params;

/* Scores of the winning candidate and of the best candidate belonging to a different child. */
typedef struct ref_select_info {
    float best;
    float second;
    int32_t n_candidates; /* children that took part */
    int32_t near_tie;     /* |best-second| <= 1e-6 * max(|best|,|second|) */
} ref_select_info;

float ref_combined_value(const ref_tree *t, int32_t node, float rave_k);
/* The two per-child scores of selectChild: first loop and second loop. */
void ref_child_scores(const ref_tree *t, int32_t parent, int32_t child, const ref_params *p,
                      float *score_first, float *score_second);
int32_t ref_ceil_sqrt(int32_t n);
int32_t ref_select_child(const ref_tree *t, int32_t node, const ref_params *p, ref_select_info *info);

void ref_add_vl(ref_tree *t, int32_t node, int32_t amount);
void ref_remove_vl1(ref_tree *t, int32_t node);
void ref_remove_vl(ref_tree *t, int32_t node, int32_t amount);
void ref_update(ref_tree *t, int32_t node, float value);

/* paths: [B][max_depth+1] node ids (row per traversal), unused entries -1.
 * near_tie_depth (may be NULL): first selection step of the traversal with a near tie, else -1. */
int ref_select_batch(ref_tree *t, const int32_t *roots, int32_t B, const ref_params *p,
                     int32_t *paths, int32_t *path_len, int32_t *leaf, int32_t *near_tie_depth);
void ref_apply_vl_paths(ref_tree *t, const int32_t *paths, const int32_t *path_len, int32_t B,
                        int32_t stride, int32_t amount);
void ref_revert_vl_paths(ref_tree *t, const int32_t *paths, const int32_t *path_len, int32_t B,
                         int32_t stride, int32_t amount);
void ref_backup_batch(ref_tree *t, const int32_t *paths, const int32_t *path_len,
                      const float *values, int32_t B, int32_t stride, int32_t amount);
/* Leaf gather: the move list replayed on the root state, actions[B][max_depth], unused -1. */
void ref_gather_actions(const ref_tree *t, const int32_t *paths, const int32_t *path_len,
                        int32_t B, int32_t stride, int32_t *actions);

/* Leaf expansion as the backup phase of executeBatchedTreeSearch does it for the leaves of a
 * batch (src/mcts/mcts_engine_batch_tree_simple.cpp:249-259): MCTSNode::expand
 * (src/mcts/mcts_node.cpp:238-436) followed by setPriorProbabilities (:512-593).
 *   - traversal t offers the legal moves moves[move_begin[t] .. move_begin[t+1]) of its leaf;
 *     an empty list is a terminal state: the node stays a leaf (:257-259, :282-284);
 *   - a leaf reached by several traversals is expanded once, by the first of them in index
 *     order that offers moves (is_expanded_ compare-exchange, :263-265: the first caller
 *     wins; one thread in index order is the deterministic schedule);
 *   - a node that already has children is left alone (same compare-exchange);
 *   - at most 1000 moves are used (max_reasonable_moves, :289-293);
 *   - one child per move, in the order given (the reference shuffles the moves with a
 *     random_device seed, :357-364, so every order is one of its outcomes), with zero
 *     statistics, action = the move (:396-404);
 *   - priors: without a policy the uniform 1/children of expand (:426-429); with a policy
 *     row of action_space entries, clamp(policy[move], 0, 1), and 0.01 for a move outside
 *     the action space (:537-558).
 * The arrays hold room for `capacity` nodes; new ids are handed out in traversal order from
 * n_nodes on.  first_child[t] (may be NULL) = first new id for the traversal whose list was
 * used, else -1.  Returns the node count afterwards, or -1 when capacity would be exceeded
 * (nothing is changed then).
 * PARITY UNPINNED where the reference is random (child order) or silent (nothing in its tests
 * fixes the priors); pinned: children = legal moves, terminal stays leaf, actions in range
 * (tests/mcts/mcts_node_test.cpp:124-170), and the prior rules restated above. */
int64_t ref_expand_batch(int64_t n_nodes, int64_t capacity, int32_t *N, float *W, float *P, int32_t *VL,
                         int32_t *rN, float *rW, int32_t *child_begin, int32_t *child_count, int32_t *action,
                         uint32_t *legal, const int32_t *leaf, int32_t B, const int32_t *move_begin,
                         const int32_t *moves, const float *policy, int32_t action_space, int32_t *first_child);

/* The same with everything expand() and setPriorProbabilities() look at: a policy vector of its own
 * length per traversal (policy_begin[t] .. policy_begin[t+1]: empty = setPriorProbabilities is not
 * called, action_space values = by action, as many values as children = by child index, any other
 * length = uniform, :537-584) and progressive widening (use_pw, cpw, kpw: only the first
 * ref_widened_children(...) of the offered moves become children, :296-341; the incremental branch
 * of expand() is unreachable behind the compare-exchange of :264).
 * Pinned: closed forms of the child count (tests/test_oracle_expand.py), the reference-test facts
 * (children >= 4 and <= legal moves, tests/mcts/progressive_widening_test.cpp:124-139). */
int32_t ref_widened_children(int32_t legal, int32_t visits, int32_t use_pw, float cpw, float kpw);
int64_t ref_expand_batch_ex(int64_t n_nodes, int64_t capacity, int32_t *N, float *W, float *P, int32_t *VL,
                            int32_t *rN, float *rW, int32_t *child_begin, int32_t *child_count, int32_t *action,
                            uint32_t *legal, const int32_t *leaf, int32_t B, const int32_t *move_begin,
                            const int32_t *moves, const int32_t *policy_begin, const float *policy,
                            int32_t action_space, int32_t use_pw, float cpw, float kpw, int32_t *first_child);

/* Dirichlet noise on the root's priors from caller-drawn gamma samples (see ref_cpu.c). */
int32_t ref_add_root_noise(ref_tree *t, int32_t root, const float *gamma, int32_t n_gamma, float epsilon);

/* MCTSEngine::getActionProbabilities (src/mcts/mcts_engine_tree.cpp:388-465): the search
 * result's move probabilities from the root's children.  counts = float(N_child);
 * temperature < 0.01: 1 for the FIRST child with the largest count, 0 elsewhere; else
 * (count / max_count) ^ (1 / temperature) for count > 0, normalised by their sum in child
 * order; uniform 1 / children when every count is 0 (or the sum is 0).  The result is laid
 * out over the action space: out[action_i] = probability_i for 0 <= action_i < action_space
 * (a later child with the same action overwrites an earlier one), 0 elsewhere.  Returns the
 * number of children, 0 when the root has none (the reference returns an empty vector; out
 * is left all zero).  Slots whose legal bit is clear are not children. */
int32_t ref_action_probabilities(const ref_tree *t, int32_t root, float temperature, int32_t action_space,
                                 float *out);

/* The RAVE part of MCTSEngine::backPropagate (src/mcts/mcts_engine_tree.cpp:288-331, with
 * MCTSNode::updateRAVE, src/mcts/mcts_node.cpp:631-643), for a batch of paths in index order.
 * The reference only runs it from a search loop that is not dispatched any more; it is
 * restated for completeness.  path_actions = the actions of all nodes of the path that have
 * one (action != -1, :296-300).  Going from the leaf to the root, with the value's sign
 * flipped per ply as in the backup, every child of the path node whose action occurs in
 * path_actions gets rave_count += 1 and rave_value_sum += the node's signed value, once per
 * child (:310-324).  Slots whose legal bit is clear are not children.  Touches rN / rW only. */
void ref_rave_backup_batch(ref_tree *t, const int32_t *paths, const int32_t *path_len, const float *values,
                           int32_t B, int32_t stride);

/* Tree reuse between moves (MCTSEngine::searchWithTreeReuse,
 * src/mcts/mcts_engine_search.cpp:1029-1075): the new root is the FIRST child of the old root
 * whose action is last_action (:1041-1043, children in order); everything else of the old
 * tree is dropped.  Returns the child's id, or -1 when there is none (the reference then
 * falls back to a fresh search). */
int32_t ref_reroot_child(const ref_tree *t, int32_t root, int32_t last_action);
/* The subtree of new_root renumbered so that it fills ids 0..k-1: breadth-first, siblings
 * contiguous and in their old order (so selections come out the same), new_root = 0.
 * old_of_new[i] receives the old id of new node i (room for n_nodes entries); returns k.
 * (The reference keeps pointers, so it has no numbering to preserve: this only reclaims the
 * arrays of the dropped siblings.) */
int64_t ref_compact_order(const ref_tree *t, int32_t new_root, int32_t *old_of_new);

/* Open-addressing table: 2^log2_slots slots of 16 bytes, linear probing,
 * home slot = (key * 0x9E3779B97F4A7C15) >> (64 - log2_slots), empty key = ~0. */
typedef struct ref_tt_slot {
    uint64_t key;
    int32_t node;
    int32_t depth;
} ref_tt_slot;

void ref_tt_clear(ref_tt_slot *slots, int32_t log2_slots);
/* 0 stored, 1 key already present (first entry kept), -1 table full, -2 reserved key */

/* What PHMapTranspositionTable::Entry keeps for its replacement policy, beside the slots. */
typedef struct ref_tt_meta {
    uint32_t visits;
    float value;
    uint32_t last_access;
    int32_t reserved;
} ref_tt_meta;
/* store() with the replacement policy and lookup() with its time stamp, for batches (see ref_cpu.c).
 * PARITY UNPINNED against the reference (its table is phmap v1.3.8, absent, and its clock depends on
 * the thread schedule); pinned against a literal Python restatement of store / lookup over a dict
 * (tests/test_oracle_tt.py), which agrees wherever a key occurs once per call or is stored without
 * visits, the reference's two call sites. */
int ref_tt_store_batch(ref_tt_slot *slots, ref_tt_meta *meta, int32_t log2_slots, const ref_tree *t,
                       const uint64_t *keys, const int32_t *nodes, const int32_t *depths, int64_t n, uint32_t t0,
                       float threshold, int32_t *counts);
int64_t ref_tt_lookup_batch(const ref_tt_slot *slots, ref_tt_meta *meta, int32_t log2_slots, const uint64_t *keys,
                            int64_t n, int32_t min_depth, uint32_t t0, int32_t *out_node);
int ref_tt_insert(ref_tt_slot *slots, int32_t log2_slots, uint64_t key, int32_t node, int32_t depth);
/* out_node[i] = node stored under keys[i] with depth >= min_depth, else -1; returns hits */
int64_t ref_tt_probe(const ref_tt_slot *slots, int32_t log2_slots, const uint64_t *keys, int64_t n,
                     int32_t min_depth, int32_t *out_node);

/* The traversal loop with the transposition table on, redirects included (see ref_cpu.c): alias[n_nodes]
 * (-1 = the slot holds its own node) is read and updated; paths [B][max_depth+1], moves [B][max_depth]
 * (may be NULL); counts[6].  The table's clock is the reference's on one thread (it ticks on a store that
 * finds its key and on a lookup that hits); with several threads the reference's stamps depend on the
 * schedule.  The loop, the clock included, is pinned by a literal restatement over node objects with
 * children lists and a dictionary as the table (tests/test_oracle_redirect.py). */
int ref_select_redirect_batch(ref_tree *t, int32_t *alias, const int32_t *roots, int32_t B, const ref_params *p,
                              ref_tt_slot *slots, ref_tt_meta *meta, int32_t log2_slots, uint32_t t0, float threshold,
                              const uint64_t *node_key, int32_t *paths, int32_t *path_len, int32_t *leaf,
                              int32_t *moves, int32_t *counts);

/* ---- position keys: utils::ZobristHash tables and GomokuState::getHash() of a replayed path ---- */
typedef struct ref_mt64 {
    uint64_t mt[312];
    int idx;
} ref_mt64;
void ref_mt64_seed(ref_mt64 *g, uint64_t seed);
uint64_t ref_mt64_next(ref_mt64 *g);
/* piece[n_piece][board_size * board_size], player[n_players]; -1 for arguments the constructor rejects
 * and for seed 0 (the reference then seeds from the clock) */
int ref_zobrist_tables(int32_t board_size, int32_t n_piece, int32_t n_players, uint32_t seed, uint64_t *piece,
                       uint64_t *player);
/* board[cell] = 0 empty, 1 BLACK, 2 WHITE; current_player 1 or 2; piece[side * piece_stride + cell] */
uint64_t ref_position_key(const int8_t *board, int32_t cells, const uint64_t *piece, int64_t piece_stride,
                          const uint64_t *player, int32_t current_player);
/* paths row-major [B][stride]; root_boards [B][cells]; root_player [B] in {1, 2}; returns bad paths */
int32_t ref_leaf_keys(const ref_tree *t, const int32_t *paths, const int32_t *path_len, int32_t B, int32_t stride,
                      const int8_t *root_boards, const int32_t *root_player, int32_t cells, const uint64_t *piece,
                      int64_t piece_stride, const uint64_t *player, uint64_t *out);

#ifdef __cplusplus
}
#endif
#endif
