/*
 * omk_forest.h -- C ABI of the device-resident search forest (MI355X / gfx950).
 *
 * The library replaces the pointer tree of the reference (class MCTSNode,
 * include/mcts/mcts_node.h:20-199) by per-node arrays in HBM and the inner loops of
 * MCTSEngine::executeBatchedTreeSearch (src/mcts/mcts_engine_batch_tree_simple.cpp)
 * by HIP kernels.  Each entry point names the reference code it stands for.
 *
 * Conventions
 *   - every function returns an omk_status (0 = OK, negative = error); no C++
 *     exception crosses this boundary; omk_last_error() gives the message of the
 *     calling thread's last failure;
 *   - handles are opaque and own their device memory; the caller owns every
 *     host buffer it passes;
 *   - pointers named h_* are host pointers, d_* are device pointers;
 *   - all work of a forest is enqueued on one HIP stream (its own by default,
 *     see omk_forest_set_stream); calls that return data to the host wait for it;
 *   - one host thread drives a forest at a time.
 *
 * Node ids are int32 indices into the arrays; the children of node v are the ids
 * child_begin[v] .. child_begin[v]+child_count[v]-1 (their order is the order of the
 * reference's children_ vector, so "lowest index wins a tie" means the same thing).
 */
#ifndef OMK_FOREST_H
#define OMK_FOREST_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum omk_status {
    OMK_OK = 0,
    OMK_ERR_INVALID = -1,     /* bad argument                                   */
    OMK_ERR_HIP = -2,         /* a HIP runtime call failed                      */
    OMK_ERR_CAPACITY = -3,    /* larger than the handle was created for         */
    OMK_ERR_STRUCTURE = -4,   /* the uploaded arrays do not describe a forest   */
    OMK_ERR_UNSUPPORTED = -5, /* valid request this build has no kernel for     */
    OMK_ERR_STATE = -6        /* call order (e.g. backup before any select)     */
} omk_status;

#define OMK_MAX_FANOUT 1024 /* children per node the selection kernels hold in registers */

typedef struct omk_forest omk_forest;
typedef struct omk_batch omk_batch;
typedef struct omk_tt omk_tt;

/* Host view of the per-node arrays: the flattened fields of MCTSNode
 * (include/mcts/mcts_node.h:154-178). */
typedef struct omk_soa_view {
    int64_t n_nodes;
    int32_t *N;                 /* visit_count_                                  */
    float *W;                   /* value_sum_                                    */
    float *P;                   /* prior_probability_                            */
    int32_t *VL;                /* virtual_loss_count_                           */
    int32_t *rN;                /* rave_count_      (NULL unless the forest has RAVE) */
    float *rW;                  /* rave_value_sum_  (NULL unless the forest has RAVE) */
    const int32_t *child_begin; /* children_: first child id                     */
    const int32_t *child_count; /* children_.size(); 0 = isLeaf()                */
    const int32_t *action;      /* action_ (NULL: the node id stands in)         */
    const uint32_t *legal;      /* optional bit per node id (bit i of word i/32): 0 = the slot
                                   holds no child and never takes part in a selection */
    const uint64_t *hash;       /* optional position key of the node's state (getHash()) */
} omk_soa_view;

typedef struct omk_forest_desc {
    int64_t capacity_nodes;
    int32_t device;   /* HIP device ordinal */
    int32_t has_rave; /* allocate rN / rW   */
} omk_forest_desc;

/* MCTSSettings fields read on this path (include/mcts/mcts_engine.h:81-112). */
typedef struct omk_select_params {
    float c_puct;         /* exploration_constant                                  */
    int32_t virtual_loss; /* virtual_loss                                          */
    int32_t use_rave;     /* use_rave: second scan of selectChild blends RAVE      */
    float rave_k;         /* rave_constant                                         */
    int32_t pw;           /* selection-time progressive widening: only the top
                             ceil(sqrt(N_parent)) children by prior take part.
                             Needs children stored in prior-descending order.      */
} omk_select_params;

/* Device pointers of a batch, for consumers that stay on the GPU. Level-major:
 * the node of traversal t at depth d is d_paths[d * stride + t]. */
typedef struct omk_batch_dev {
    int32_t *d_paths;
    int32_t *d_path_len; /* nodes on the path (selection steps + 1) */
    int32_t *d_leaf;
    float *d_values;
    int32_t stride;
    int32_t max_depth;
    int32_t n_traversals;
} omk_batch_dev;

const char *omk_last_error(void);
int omk_version(void);

/* ---- forest: replaces the MCTSNode allocations (MCTSNode::create, mcts_node.cpp:68-75) ---- */
int omk_forest_create(const omk_forest_desc *desc, omk_forest **out);
int omk_forest_destroy(omk_forest *f);
/* Use the caller's hipStream_t (NULL restores the forest's own stream). */
int omk_forest_set_stream(omk_forest *f, void *hip_stream);
/* The hipStream_t the forest's work is enqueued on (to record events on it). */
int omk_forest_get_stream(omk_forest *f, void **hip_stream_out);
/* Checks that the arrays describe a forest (ranges in bounds, every node the child of at
 * most one parent, fan-out <= OMK_MAX_FANOUT) and copies them to the device.  Uploading the same
 * child ranges again (statistics put back) leaves batches usable; after an upload of another
 * structure their roots and paths are stale: OMK_ERR_STATE until omk_batch_set_roots. */
int omk_forest_upload(omk_forest *f, const omk_soa_view *h_view);
/* Copies N, W, P, VL (and rN, rW) back; structure pointers of the view are ignored. */
int omk_forest_download(omk_forest *f, omk_soa_view *h_view);
/* Nodes the forest holds now (it grows with omk_expand_batch) and the room it was created
 * with.  Either pointer may be NULL. */
int omk_forest_node_count(omk_forest *f, int64_t *h_nodes, int64_t *h_capacity);
/* Copies the structure back: first child id, child count (MCTSNode::getChildren().size(),
 * 0 = isLeaf, src/mcts/mcts_node.cpp:442-444) and action (getAction) of every node; n_nodes
 * must be the current node count; any pointer may be NULL. */
int omk_forest_download_structure(omk_forest *f, int64_t n_nodes, int32_t *h_child_begin, int32_t *h_child_count,
                                  int32_t *h_action);
int omk_sync(omk_forest *f);

/* Host-side re-layout of a forest whose nodes keep one slot per action and a legal mask (a board
 * layout: 362 slots per expanded Go node, a bit per slot) into the layout of the reference itself,
 * whose children_ vector holds the legal moves only (MCTSNode::expand, src/mcts/mcts_node.cpp:238-436):
 * the nodes whose bit is set, in their old order, renumbered 0 .. count-1, child ranges shrunk to
 * match, the slot index kept as the node's action.  A selection on the result visits the same
 * children in the same order (ties still go to the lowest child), reads half the cache lines and
 * takes four rounds of 64 lanes where a 362-slot node takes six; node ids in paths and leaves are
 * the new ones, new_to_old maps them back.  No GPU call; omk_forest_upload takes the result
 * (legal = NULL).
 * omk_soa_count_legal: how many nodes the result has (n_nodes when the view has no mask).
 * omk_soa_compact_legal: fills the caller's arrays of that many elements (rN, rW, hash: NULL when
 * the view has none or they are not wanted) and the two id maps (old_to_new: n_nodes entries, -1 for
 * an empty slot; new_to_old: count entries; either may be NULL).  action receives the view's action
 * of every kept node or, when the view has none, the node's slot in its parent's range (-1 for a
 * node that is nobody's child). */
int64_t omk_soa_count_legal(const omk_soa_view *h_view);
int omk_soa_compact_legal(const omk_soa_view *h_view, int64_t count, int32_t *N, float *W, float *P, int32_t *VL,
                          int32_t *rN, float *rW, int32_t *child_begin, int32_t *child_count, int32_t *action,
                          uint64_t *hash, int32_t *old_to_new, int32_t *new_to_old);

/* ---- batch: the per-search buffers of executeBatchedTreeSearch
 *      (leaf_nodes / paths / leaf_states, mcts_engine_batch_tree_simple.cpp:41-57) ---- */
int omk_batch_create(omk_forest *f, int32_t max_traversals, int32_t max_depth, omk_batch **out);
int omk_batch_destroy(omk_batch *b);
/* Traversal t starts at h_roots[t] (the reference: every simulation starts at root_,
 * mcts_engine_batch_tree_simple.cpp:86-92).  Distinct roots must head disjoint trees. */
int omk_batch_set_roots(omk_batch *b, const int32_t *h_roots, int32_t n_traversals);
int omk_batch_set_values(omk_batch *b, const float *h_values, int32_t n); /* NetworkOutput::value of each leaf */
int omk_batch_device(omk_batch *b, omk_batch_dev *out);

/* Phase 1 of executeBatchedTreeSearch (mcts_engine_batch_tree_simple.cpp:73-185): for
 * every traversal, in traversal-index order semantics, descend while the node is expanded:
 * MCTSNode::selectChild (mcts_node.cpp:90-236, with getCombinedValue :657-678 when use_rave),
 * then addVirtualLoss(virtual_loss) on the selected child (mcts_node_virtual_loss.cpp:15-20).
 * Results stay on the device (omk_batch_read / omk_batch_device). Asynchronous. */
int omk_select_batch(omk_batch *b, const omk_select_params *params);

/* Phase 3 (mcts_engine_batch_tree_simple.cpp:276-281) on the paths of the last select:
 * leaf to root, MCTSNode::update(value) (mcts_node_virtual_loss.cpp:54-71), then
 * revertVirtualLoss(virtual_loss) (:32-42), value = -value.  Asynchronous. */
int omk_backup_batch(omk_batch *b, int32_t virtual_loss);
/* removeVirtualLoss(virtual_loss) on every node of the paths of the last select. */
int omk_revert_vl(omk_batch *b, int32_t virtual_loss);

/* The same three node operations over caller-supplied device paths (level-major, node of
 * traversal t at depth d = d_paths[d*stride+t], d < d_path_len[t]); atomics, any paths. */
int omk_apply_vl_paths(omk_forest *f, const int32_t *d_paths, const int32_t *d_path_len, int32_t n,
                       int32_t stride, int32_t max_len, int32_t virtual_loss);
int omk_revert_vl_paths(omk_forest *f, const int32_t *d_paths, const int32_t *d_path_len, int32_t n,
                        int32_t stride, int32_t max_len, int32_t virtual_loss);
int omk_backup_paths(omk_forest *f, const int32_t *d_paths, const int32_t *d_path_len,
                     const float *d_values, int32_t n, int32_t stride, int32_t max_len, int32_t virtual_loss);

/* Dirichlet noise on the priors of `root`'s children (MCTSEngine::addDirichletNoise,
 * src/mcts/mcts_engine_eval.cpp:78-110): the caller draws one gamma(alpha, 1) sample per
 * child with its own generator, as the reference does with std::gamma_distribution on the
 * engine's random engine (:83-90); the library normalises them (their float sum in order;
 * uniform 1/children when it is not positive) and sets
 * prior = (1 - epsilon) * prior + epsilon * noise, child by child in the reference's
 * order.  n_gamma must be the number of children (legal slots).  A root without children
 * is left alone.  Waits for the stream; the arithmetic is done on the host. */
int omk_forest_add_root_noise(omk_forest *f, int32_t root, const float *h_gamma, int32_t n_gamma, float epsilon);

/* The search result's move probabilities (MCTSEngine::getActionProbabilities,
 * src/mcts/mcts_engine_tree.cpp:388-465) from the visit counts of `root`'s children, laid
 * out over the action space: temperature < 0.01 puts 1 on the first child with the largest
 * count; otherwise (count / max_count) ^ (1 / temperature) normalised, uniform when every
 * count is 0.  Waits for the stream, reads the children's counts and actions back and does
 * the arithmetic on the host, in the reference's order (it is a few hundred numbers per
 * search).  h_children (may be NULL) receives the number of children; with none the output
 * is all zero. */
int omk_forest_action_probabilities(omk_forest *f, int32_t root, float temperature, int32_t action_space,
                                    float *h_probabilities, int32_t *h_children);

/* Tree reuse between moves (MCTSEngine::searchWithTreeReuse,
 * src/mcts/mcts_engine_search.cpp:1029-1075): the node to search from after `last_action` was
 * played is the first child of `root` with that action (-1 in *h_child when there is none:
 * the reference then starts a fresh search).  Node ids stay valid: pass the child to
 * omk_batch_set_roots and go on. */
int omk_forest_reroot_child(omk_forest *f, int32_t root, int32_t last_action, int32_t *h_child);
/* Drops everything but the subtree of new_root (what the reference achieves by clearing the
 * siblings' children, :1049-1055) and renumbers that subtree to ids 0..k-1: breadth-first,
 * siblings contiguous in their old order, new_root = 0, so selections come out the same.
 * *h_nodes_after = k; h_old_of_new (NULL or room for the old node count) receives the old id
 * of every new node.  Paths of earlier selections, roots of batches and node ids stored in
 * transposition tables refer to the old numbering: set roots again (a batch refuses to select,
 * back up, expand or read with OMK_ERR_STATE until then), clear the tables.  All
 * of it runs on the device: the renumbering level by level (child counts of a level, an
 * exclusive scan, the children's ids written to the next level), then one gather per array;
 * the host only reads the size of every level. */
int omk_forest_compact(omk_forest *f, int32_t new_root, int64_t *h_nodes_after, int32_t *h_old_of_new);

/* omk_forest_compact for callers that cannot allocate device memory (code under HIP graph
 * capture around it, tight serving loops, harnesses that forbid hipMalloc); it has no counterpart
 * in the reference.  Same arguments, same result, but every piece of device scratch memory (the
 * breadth-first order, the per-level counts and their scan, the staging array the fields pass
 * through) lives in one array inside the library that each GPU holds for the life of the process
 * (about 25 MiB), and the call makes no hipMalloc / hipFree.  Limit: the forest may hold at most
 * 2^20 = 1048576 nodes when it is called (OMK_ERR_CAPACITY beyond that, and nothing is changed).
 * All calls on one GPU share that array: two calls that overlap in time on the same GPU, from
 * whatever forests or threads, race; calls one after another need no clearing in between. */
int omk_forest_compact_static(omk_forest *f, int32_t new_root, int64_t *h_nodes_after, int32_t *h_old_of_new);

/* Leaf expansion for the leaves of the last selection: MCTSNode::expand
 * (src/mcts/mcts_node.cpp:238-436) followed by setPriorProbabilities (:512-593), as the backup
 * phase does before it backs the values up (src/mcts/mcts_engine_batch_tree_simple.cpp:249-259).
 * The game rules stay on the host: simulation t offers the legal moves
 * h_moves[h_move_begin[t] .. h_move_begin[t+1]) of its leaf state (the state it replayed from
 * omk_batch_read); an empty list means a terminal state, the node stays a leaf.  A leaf
 * reached by several simulations is expanded once, with the list of the first of them in
 * index order that offers moves; a node that already has children (the selection stopped at it
 * because of the depth bound) is left alone and takes no ids; at most
 * 1000 moves are used (the reference's limit).  One child per move in the order given (the
 * reference shuffles with a random seed: every order is one of its outcomes), zero
 * statistics, action = the move.  Priors: h_policy NULL -> 1 / children (expand's uniform
 * prior); else row t of h_policy has action_space entries and the prior is
 * clamp(policy[move], 0, 1), or 0.01 for a move outside the action space.  New node ids are
 * handed out from the current node count on, in simulation order; OMK_ERR_CAPACITY (and no
 * change) when the forest's capacity would be exceeded.  h_first_child (NULL or [n]): first
 * new id for the simulation whose list was used, else -1.  Waits for the stream. */
int omk_expand_batch(omk_batch *b, const int32_t *h_move_begin, const int32_t *h_moves, const float *h_policy,
                     int32_t action_space, int32_t *h_first_child);

/* The same with everything MCTSNode::expand and setPriorProbabilities look at.
 *   - Progressive widening (expand(use_progressive_widening, cpw, kpw), the MCTSSettings fields of
 *     include/mcts/mcts_engine.h:98-103, default on, c = 2, k = 0.5): a leaf of N visits that is
 *     offered L moves gets the first min(L, size_t(max(8.0f, float(cpw * pow(N + 1, kpw))))) of them
 *     (at least one) as children (src/mcts/mcts_node.cpp:296-341; the reference shuffles first, so
 *     any L-subset in any order is one of its outcomes).  The branch of expand() that would add
 *     children to a node that already has some is unreachable in the reference (the compare-exchange
 *     on is_expanded_ at :264 returns first): here, too, such a node is left alone.
 *   - One policy vector per simulation, of its own length (h_policy_begin[t] .. h_policy_begin[t+1]
 *     into h_policy; both NULL = none): empty = setPriorProbabilities is not called and expand's
 *     uniform 1 / children stays (mcts_engine_batch_tree_simple.cpp:256-258); action_space values =
 *     clamp(policy[move], 0, 1), 0.01 for a move outside the action space (:537-560); as many values
 *     as children = clamp(policy[i], 0, 1) by child index (:561-575); any other length = uniform
 *     1 / children (:576-584). */
typedef struct omk_expand_params {
    int32_t action_space;             /* IGameState::getActionSpaceSize() of the leaf states */
    int32_t use_progressive_widening; /* MCTSSettings::use_progressive_widening */
    float progressive_widening_c;     /* MCTSSettings::progressive_widening_c */
    float progressive_widening_k;     /* MCTSSettings::progressive_widening_k */
} omk_expand_params;
int omk_expand_batch_ex(omk_batch *b, const int32_t *h_move_begin, const int32_t *h_moves, const int32_t *h_policy_begin,
                        const float *h_policy, const omk_expand_params *params, int32_t *h_first_child);

/* The RAVE statistics of MCTSEngine::backPropagate (src/mcts/mcts_engine_tree.cpp:288-331 with
 * MCTSNode::updateRAVE, src/mcts/mcts_node.cpp:631-643) for the paths of the last selection
 * and the values of omk_batch_set_values: every child of a path node whose action occurs
 * among the actions of the path's nodes gets rave_count += 1 and rave_value_sum += the
 * node's signed value (sign as in the backup), once per child.  The reference's live
 * batched loop never calls this (its RAVE counts stay zero); it is offered for engines
 * that do.  Needs a forest created with RAVE arrays.  Asynchronous on the forest's stream. */
int omk_backup_rave_batch(omk_batch *b);

/* Leaf gather (mcts_engine_batch_tree_simple.cpp:114,166-184): waits for the stream and
 * returns, per traversal, the path (row of max_depth+1 ids, -1 padded), its length, the
 * leaf node and the move list to replay on a clone of the root state (row of max_depth
 * actions, -1 padded).  Any pointer may be NULL. */
int omk_batch_read(omk_batch *b, int32_t *h_paths, int32_t *h_path_len, int32_t *h_leaf, int32_t *h_actions);
/* Traversals of the last select that stopped at max_depth on an expanded node. */
int omk_batch_truncated(omk_batch *b, int32_t *h_count);
/* How the last select did its work, 16 counters: [0] multi-visitor nodes processed,
 * [1] of these settled by the parallel paths, [2] visitors settled by them, [3] visitors
 * settled one at a time, [4] nodes replayed one visitor at a time because the parallel
 * path's exactness checks did not hold, [5] threshold probes, [6] single-visitor selection
 * steps, [7] nodes settled by merging a few entries of other children into the list of the child
 * that takes nearly every visitor, [8] when the first block of the persistent launch started,
 * [9] when its last team of wavefronts left, [10] when its last walker left (low 31 bits of the
 * device's 100 MHz clock; these three are kept whether or not the counters are on), [11] the number
 * of walks of lone visitors inside that launch, [12] nodes of more than 64 child slots settled through
 * the few children that can be chosen at all, one per lane (RAVE layouts), [13..14] unused (0), [15] nodes
 * cut into slices for several wavefronts.  (Nodes taken by the walk down one-winner nodes count in [0]..[2].) */
int omk_batch_stats(omk_batch *b, int32_t *h_stats16);
/* The counters above cost one atomic per processed node (and per single-visitor step), all on
 * the same few addresses, so they are off unless switched on here (enabled != 0); with
 * them off omk_batch_stats returns zeros.  Diagnostics only; no counterpart in the reference. */
int omk_batch_set_stats(omk_batch *b, int32_t enabled);
/* Measurement aid, no counterpart in the reference: the timeline of the last select, switched on
 * with omk_batch_set_trace before that select.  One record of twelve int64 per piece of work: start
 * and end on the GPU's 100 MHz clock, visitors | depth << 32 | kind << 60 (0 a node settled as a
 * whole, 1 a slice of a heavy node, 2 a part of its partition, 3 a node published before its visitor
 * list was complete, 4 one boundary between two slices of a heavy node worked out ahead of time, 5 a node
 * whose visitors all follow one child, taken by the walk down such nodes,
 * 6 the walk of a lone visitor inside the persistent launch), node | number << 32 (number: for a slice
 * or a part of a heavy node, which one of how many: index | count << 16), then, for a slice of a heavy node,
 * word 4 = time of its boundaries | time of its batches << 32 (100 MHz clock) and word 5 = entries its
 * boundaries put in its batch (-1: it searched for the batch itself) | visitors it settled << 32; the other
 * words are 0.
 * h_trace has room for max_entries records; the records live in the staging memory of
 * omk_batch_read until the next call of it. */
int omk_debug_trace(omk_batch *b, long long *h_trace, int32_t max_entries, int32_t *h_n);
/* Switches the recording of that timeline on or off for the selects that follow (off by default: a
 * record costs one atomic and twelve stores per work item). */
int omk_batch_set_trace(omk_batch *b, int32_t enabled);
/* The multi-visitor selection kernel is persistent: its wavefronts wait for work items that
 * other wavefronts publish.  Every wait is bounded; a wavefront that polls `polls` times in
 * vain raises an abort flag, all wavefronts leave, and omk_batch_read reports OMK_ERR_STATE
 * for that selection (its paths are incomplete; upload the statistics again before the next
 * one).  The default (about four million polls, seconds) is never reached in normal
 * operation; tests of the error path set a tiny limit.  No counterpart in the reference. */
int omk_batch_set_spin_limit(omk_batch *b, int32_t polls);
/* The ready marks of the scheduler's queues are the number of the select call on the batch, which starts
 * over (all marks cleared) shortly before 2^30 calls: some days of continuous search.  A test cannot wait
 * for that; this sets the number of the call made last (0 <= count < 2^30), so that the next calls cross
 * the point.  Only between a batch's selections (the marks in memory belong to earlier numbers: moving the
 * count BACK to a number already used leaves stale marks that look fresh, so go forward only).  No
 * counterpart in the reference. */
int omk_debug_set_select_count(omk_batch *b, int32_t count);

/* ---- transposition table: the lookup/store call sites of
 *      mcts_engine_batch_tree_simple.cpp:126,141 (PHMapTranspositionTable::store / lookup,
 *      phmap_transposition_table.cpp:51-117) over an open-addressing table in HBM ---- */
typedef struct omk_tt_slot {
    uint64_t key; /* ~0 = empty */
    int32_t node;
    int32_t depth;
} omk_tt_slot;

/* Position key of the state every selected leaf stands for: what the traversal loop obtains by
 * cloning the root state, replaying the move list and calling getHash()
 * (mcts_engine_batch_tree_simple.cpp:119-124 and :133-137), for a game whose stones stay where they
 * are placed and whose sides alternate (GomokuState::compute_hash_signature_internal,
 * src/games/gomoku/gomoku_state.cpp:947-957: the piece keys of all stones and the key of the side
 * to move, XORed).  The caller passes the tables of the game's utils::ZobristHash
 * (src/utils/zobrist_hash.cpp:9-36; they are seeded from the clock there, so they are the
 * caller's): d_piece_keys[p * cells + action] = getPieceHash(p, action) for the two sides,
 * d_player_keys[p] = getPlayerHash(p); and per traversal the root state's getHash() and its side to
 * move (0 or 1 = current_player - 1).  d_out[t] = key of the leaf's state, ready for omk_tt_probe /
 * omk_tt_insert.  All pointers are device memory; a move outside [0, cells) is an error.  A game
 * with captures (Go) cannot be keyed from the move list alone and keeps its keys in the forest
 * (omk_soa_view.hash, omk_tt_probe_leaves). */
int omk_batch_leaf_keys(omk_batch *b, const uint64_t *d_piece_keys, int32_t cells, const uint64_t *d_player_keys,
                        const uint64_t *d_root_keys, const int32_t *d_root_players, uint64_t *d_out);

/* Position keys of single nodes: hash[h_nodes[i]] = h_keys[i] (host arrays).  For a game whose keys cannot
 * be folded from the move list (captures: Go), the keys are the game's own: the caller has the state of
 * every leaf it evaluates (the clone with the moves replayed, mcts_engine_batch_tree_simple.cpp:170-178)
 * and passes state->getHash() (include/core/igamestate.h) for the leaf's node.  A forest uploaded without
 * keys gets the array on the first call; a node that has no key yet (all of them then, and every node that
 * omk_expand_batch* adds) carries the key ~0, which the table neither stores nor finds.  Waits for the
 * stream. */
int omk_forest_set_keys(omk_forest *f, const int32_t *h_nodes, const uint64_t *h_keys, int64_t n);

int omk_tt_create(omk_forest *f, int32_t log2_slots, omk_tt **out);
int omk_tt_destroy(omk_tt *tt);
int omk_tt_clear(omk_tt *tt);
/* store(hash, node, depth) for n entries; a key already present keeps its first entry. */
int omk_tt_insert(omk_tt *tt, const uint64_t *d_keys, const int32_t *d_nodes, const int32_t *d_depths, int64_t n);
/* lookup(hash, min_depth): d_out[i] = node or -1; a successful lookup stamps the entry with its time
 * (phmap_transposition_table.cpp:107; lookup i of the call has the time t + i, see omk_tt_store). */
int omk_tt_probe(omk_tt *tt, const uint64_t *d_keys, int64_t n, int32_t min_depth, int32_t *d_out);
/* lookup of the position key of every leaf of the last select: d_out[t] = node or -1. */
int omk_tt_probe_leaves(omk_tt *tt, omk_batch *b, int32_t min_depth, int32_t *d_out);
/* PHMapTranspositionTable::store (phmap_transposition_table.cpp:51-84) for n entries: a key that is
 * not in the table gets a new entry (createEntry :202-216: node, depth as a uint16, the node's visit
 * count and value as they are now); a key that is there keeps its entry unless the new one's
 * replacement score exceeds the old one's by the threshold (:64-74, score = recency * importance,
 * include/mcts/phmap_transposition_table.h:68-72, threshold Config::replacement_threshold = 0.1).
 * Time (not the reference's: replacement decisions that hinge on recency are not pinned against it):
 * the reference advances its access counter on a store that finds the key and on a lookup that hits
 * (:64, :107), from threads that share it, so its stamps depend on the schedule; here entry i of a call
 * has the time t + i and the table's clock t advances by n per call, misses included (lookups
 * likewise).  Among the entries of one call with the same key only the first is
 * stored: the serial outcome at the reference's two call sites (a node stored from the traversal
 * has no visits, score 0, and never replaces; the leaves expanded in one step are distinct).
 * An entry with node < 0 is skipped.  h_counts (NULL or [4]): new entries, replacements, entries
 * dropped as duplicates within the call, 0.  Waits for the stream. */
int omk_tt_store(omk_tt *tt, const uint64_t *d_keys, const int32_t *d_nodes, const int32_t *d_depths, int64_t n,
                 int32_t *h_counts);
int omk_tt_set_replacement_threshold(omk_tt *tt, float threshold);
/* The transposition-table part of the traversal loop (mcts_engine_batch_tree_simple.cpp:116-162)
 * for the paths of the last select: at every step the selected child is stored under the key of
 * the state it stands for when it has no visits yet (:116-128, depth = moves so far), then the key
 * is looked up, and a node OTHER than the selected one that has visits is a transposition
 * (:141-142).  The reference then swaps the child pointer of the parent for that node (:143-156),
 * which turns the tree into a graph; this library reports the transposition and leaves the tree
 * alone: d_hits (NULL when only the counts are wanted, or device memory for n_traversals * max_depth ints, entry t * max_depth + d - 1
 * for step d of traversal t) receives that node or -1.  Keys: with d_piece_keys the game's Zobrist
 * tables as in omk_batch_leaf_keys (stone-placing games), with NULL the forest's per-node keys
 * (omk_soa_view.hash).  h_counts (NULL or [4]): new entries, replacements, duplicates within the
 * call, transpositions reported.  Waits for the stream. */
int omk_tt_traverse(omk_tt *tt, omk_batch *b, const uint64_t *d_piece_keys, int32_t cells, const uint64_t *d_player_keys,
                    const uint64_t *d_root_keys, const int32_t *d_root_players, int32_t *d_hits, int32_t *h_counts);
/* The whole traversal loop with the table on, redirects INCLUDED (mcts_engine_batch_tree_simple.cpp:88-165;
 * the redirect is :142-156 with MCTSNode::updateChildReference, mcts_node.cpp:617-630): a select for the
 * batch's roots that, at every step, stores the selected child when it has no visits, looks the position
 * up, and on a transposition (a node other than the selected one, with visits) takes the virtual loss back
 * from the selected child, re-points the parent's child slot at the transposition, adds the virtual loss
 * there and walks on from it.  Off unless called: omk_select_batch never redirects.
 *   - Exact for the reference run by one thread: the traversals are walked one after the other by a single
 *     wavefront (a re-pointed slot is seen by every later traversal, as in the serial loop).  Expect
 *     microseconds per step, not the throughput of omk_select_batch.
 *   - A re-pointed slot holds another node: selection reads that node's statistics and prior, and the move
 *     recorded for the step is that node's action (children_[i]->getAction(), :112), as in the reference.
 *   - Keys are the forest's per-node position keys (omk_soa_view.hash / omk_forest_set_keys): the key of a
 *     step is that of the node of the tree AS UPLOADED that the recorded moves lead to from the root, which
 *     is what replaying the moves on the root state gives (:119-124); where no such node exists (a move no
 *     child slot carries, a node not expanded) the step has no key and the table is not touched.
 *   - Time stamps: the table's clock advances here as the reference's access counter does on one thread: by
 *     one on a store that finds its key (phmap_transposition_table.cpp:65) and on a lookup that hits (:107).
 *   - d_moves: NULL, or device memory for max_depth * stride ints (omk_batch_dev.stride), level-major like the
 *     paths (entry (d - 1) * stride + t = the move recorded at step d of traversal t): the move list the
 *     leaf's state is rebuilt from.  It differs from the actions of the path's nodes exactly at a step that
 *     redirected.
 *   - h_counts (NULL or [5]): new entries, replacements, lookups that found an entry, redirects, steps.
 *   - A table without room for a new entry drops it and the traversals go on without it; the call then
 *     returns OMK_ERR_CAPACITY AFTER everything else is done (h_counts filled, the batch selected: read it,
 *     back it up or revert it as after any selection).  The reference's table evicts instead
 *     (enforceMemoryLimit, phmap_transposition_table.cpp:77-79): size the table for the search.
 * Paths, leaves and virtual loss are left as omk_select_batch leaves them (omk_batch_read, omk_backup_batch,
 * omk_revert_vl work on them).  Once a slot has been re-pointed the forest is a graph until the next
 * omk_forest_upload: omk_select_batch, omk_backup_rave_batch, omk_forest_add_root_noise and the compactions
 * refuse it (OMK_ERR_UNSUPPORTED); omk_forest_action_probabilities counts the visits of the nodes the root's
 * slots hold (mcts_engine_tree.cpp:395-403).  Selection-time progressive widening is refused.  Waits for the
 * stream. */
int omk_tt_select_redirect(omk_tt *tt, omk_batch *b, const omk_select_params *params, int32_t *d_moves,
                           int32_t *h_counts);
/* h_alias[n_nodes]: the node child slot s holds instead of node s, or -1 (MCTSNode::children_ after
 * updateChildReference); n_nodes must be the forest's node count. */
int omk_forest_download_redirects(omk_forest *f, int64_t n_nodes, int32_t *h_alias);
/* What an entry keeps for the replacement policy, slot by slot beside omk_tt_download. */
typedef struct omk_tt_meta {
    uint32_t visits;      /* Entry::visits */
    float value;          /* Entry::value */
    uint32_t last_access; /* Entry::last_access */
    int32_t reserved;
} omk_tt_meta;
int omk_tt_download_meta(omk_tt *tt, omk_tt_meta *h_meta);
int omk_tt_upload(omk_tt *tt, const omk_tt_slot *h_slots);
int omk_tt_download(omk_tt *tt, omk_tt_slot *h_slots);

/* ---- device memory helpers for hosts without a HIP binding of their own ---- */
int omk_dev_alloc(omk_forest *f, int64_t bytes, void **d_out);
int omk_dev_free(omk_forest *f, void *d_ptr);
int omk_dev_h2d(omk_forest *f, void *d_dst, const void *h_src, int64_t bytes);
int omk_dev_d2h(omk_forest *f, void *h_dst, const void *d_src, int64_t bytes);
/* Device-to-device copy by a plain kernel (bytes a multiple of 4), asynchronous.  It moves
 * exactly `bytes` in and `bytes` out, which is what profiler traffic counters are scaled by. */
int omk_dev_copy(omk_forest *f, void *d_dst, const void *d_src, int64_t bytes);

#ifdef __cplusplus
}
#endif
#endif
