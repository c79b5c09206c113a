// Host-side C++ adapter above the C ABI (include/omk_forest.h): the leaf-selection and
// batch-collection interface of the reference's MCTSEngine for the device-resident forest.
//
// It mirrors, phase by phase, MCTSEngine::executeBatchedTreeSearch
// (reference src/mcts/mcts_engine_batch_tree_simple.cpp:14-301):
//   selectLeafBatch      phase 1 (:73-185) + leaf gather (:166-206): one LeafItem per simulation
//   InferenceFunction    phase 2 (:212-236): the evaluator, called once per batch
//   expandLeafBatch      phase 3, first half (:249-259): expand + setPriorProbabilities of the leaves
//   backPropagateBatch   phase 3 (:276-281): update + revertVirtualLoss, sign flipped per ply
// The reference hands the evaluator cloned game states; here a LeafItem carries the leaf
// node and the move list to replay on a clone of the root state (what :170-178 does), so
// game rules stay on the host, untouched.
//
// Errors of the C ABI surface as std::runtime_error carrying omk_last_error(), which is what
// MCTSEngine::search logs and rethrows (reference src/mcts/mcts_engine_main.cpp:343-355).
#pragma once

#include <cstdint>
#include <functional>
#include <array>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/omk_forest.h"

namespace omk {

// reference include/mcts/evaluation_types.h:14-17
struct NetworkOutput {
    std::vector<float> policy;
    float value = 0.0f;
};

// The fields of MCTSSettings this path reads (reference include/mcts/mcts_engine.h:55-120).
struct MCTSSettings {
    int num_simulations = 800;
    int batch_size = 256;
    float exploration_constant = 1.4f;
    int virtual_loss = 3;
    bool use_rave = true;
    float rave_constant = 3000.0f;
    // MCTSNode::expand's progressive widening, as in the reference (default on, c = 2, k = 0.5): a leaf
    // of N visits gets min(legal, max(8, c * (N + 1)^k)) children (omk_expand_batch_ex)
    bool use_progressive_widening = true;
    float progressive_widening_c = 2.0f;
    float progressive_widening_k = 0.5f;
    // MCTSNode::expand shuffles a node's legal moves before it creates the children (reference
    // src/mcts/mcts_node.cpp:357-364); omk_expand_batch_ex keeps the order it is given, so the search
    // (omk_search.h) shuffles on the host.  Off: children in the game's own move order.
    bool shuffle_moves = true;
    bool add_dirichlet_noise = true;
    float dirichlet_alpha = 0.3f;
    float dirichlet_epsilon = 0.25f;
    float temperature = 1.0f;
    // the table of positions (reference :97-98; the slots here are 32 bytes with their policy fields)
    bool use_transposition_table = true;
    size_t transposition_table_size_mb = 128;
    // Not a field of the reference, whose traversal always follows a transposition it finds (reference
    // src/mcts/mcts_engine_batch_tree_simple.cpp:142-156).  Off: transpositions are counted and the tree stays a
    // tree (the fast selection).  On (with use_transposition_table): every batch is selected by the loop that
    // follows and re-points them as the reference does, one traversal after the other (omk_tt_select_redirect:
    // exact for the reference run by one thread, microseconds per step).
    bool follow_transpositions = false;
    // Not in the reference: only the ceil(sqrt(N_parent)) children of highest prior take part in a
    // selection (omk_select_params::pw; needs children stored by descending prior)
    bool selection_prior_widening = false;
    int max_depth = 64;  // longest path the batch buffers hold
};

// What PendingEvaluation{node, state, path} (reference include/mcts/evaluation_types.h:49-73)
// becomes when the tree lives on the device.
struct LeafItem {
    int32_t node = -1;                  // the leaf
    std::vector<int32_t> path;          // root .. leaf node ids
    std::vector<int32_t> move_sequence; // actions to replay on a clone of the root state
};

using InferenceFunction = std::function<std::vector<NetworkOutput>(const std::vector<LeafItem> &)>;
// The legal moves of every leaf's state (IGameState::getLegalMoves on the state the host
// replayed; an empty list = terminal state).  Game rules stay on the host.
using LegalMovesFunction = std::function<std::vector<std::vector<int>>(const std::vector<LeafItem> &)>;

class ForestEngine {
   public:
    ForestEngine(InferenceFunction inference_fn, const MCTSSettings &settings, int64_t capacity_nodes, int device = 0,
                 bool has_rave = false);
    ~ForestEngine();
    ForestEngine(const ForestEngine &) = delete;
    ForestEngine &operator=(const ForestEngine &) = delete;

    void uploadTree(const omk_soa_view &view);
    void downloadStatistics(omk_soa_view &view);

    // One batch: every simulation starts at `root` (reference :86-92).
    void selectLeafBatch(int32_t root, int batch_size, std::vector<LeafItem> &leaves);
    // Simulation i starts at roots[i]: independent trees searched side by side.
    void selectLeafBatch(const std::vector<int32_t> &roots, std::vector<LeafItem> &leaves);
    void backPropagateBatch(const std::vector<float> &leaf_values);
    // Expands the leaves of the last selectLeafBatch on the device as MCTSNode::expand +
    // setPriorProbabilities do (reference src/mcts/mcts_engine_batch_tree_simple.cpp:249-259): children
    // for the legal moves (the first of them under progressive widening), priors from every
    // output's own policy (by action when it has action_space entries, by child when it has as
    // many as children, uniform otherwise or when empty).  action_space <= 0: the size of the
    // first policy that is not empty.  Returns the nodes added.
    // first_child (optional): per simulation the id of the first child created from its move list, or -1.
    int64_t expandLeafBatch(const std::vector<std::vector<int>> &legal_moves, const std::vector<NetworkOutput> &outputs,
                            int action_space = 0, std::vector<int32_t> *first_child = nullptr);
    void setLegalMovesFunction(LegalMovesFunction fn) { legal_moves_fn_ = std::move(fn); }
    // SearchResult.probabilities (reference MCTSEngine::getActionProbabilities,
    // src/mcts/mcts_engine_tree.cpp:388-465): visit counts of root's children, temperature.
    std::vector<float> getActionProbabilities(int32_t root, float temperature, int action_space);
    // Dirichlet noise on the root's priors (reference MCTSEngine::addDirichletNoise,
    // src/mcts/mcts_engine_eval.cpp:78-110): one gamma(alpha, 1) sample per child, drawn by
    // the caller's generator as the reference draws them from its own.
    void addDirichletNoise(int32_t root, const std::vector<float> &gamma_samples, float epsilon);
    // Position keys of nodes from the game's own states (IGameState::getHash of the state a node stands
    // for): what the traversal loop gets by cloning and replaying (reference
    // src/mcts/mcts_engine_batch_tree_simple.cpp:119-124,133-137), for any game.
    void setPositionKeys(const std::vector<int32_t> &nodes, const std::vector<uint64_t> &keys);
    // The table's part of the traversal loop (reference :116-162) over the paths of the last
    // selectLeafBatch, keyed by the nodes' position keys: unvisited children stored, every step looked
    // up, transpositions counted (never followed).  The table is created on first use with about
    // settings.transposition_table_size_mb.  Returns {new entries, replacements, duplicates, transpositions}.
    std::array<int32_t, 4> traverseTranspositionTable();
    // With settings.follow_transpositions the selection itself is the loop with the table (reference :88-165):
    // what the last selectLeafBatch counted, {new entries, replacements, lookups that found an entry, redirects,
    // steps}.  The leaves' move_sequence is then the list of RECORDED moves (the action of the node each selected
    // slot held), which is what the reference replays; it differs from the actions of the path's nodes at a
    // step that redirected.
    std::array<int32_t, 5> lastRedirectCounts() const { return redirect_counts_; }
    bool followsTranspositions() const { return settings_.use_transposition_table && settings_.follow_transpositions; }
    int64_t nodeCount() const;
    void downloadStructure(int64_t n_nodes, int32_t *child_begin, int32_t *child_count, int32_t *action);

    // The whole loop of executeBatchedTreeSearch: batches of settings.batch_size until
    // num_simulations are done; leaves are expanded when a legal-moves function is set.
    // Returns simulations run.
    int executeBatchedTreeSearch(int32_t root);

    const MCTSSettings &settings() const { return settings_; }

   private:
    void check(int status, const char *what) const;
    void ensureBatch(int n);
    void ensureTable();

    InferenceFunction inference_fn_;
    LegalMovesFunction legal_moves_fn_;
    MCTSSettings settings_;
    omk_forest *forest_ = nullptr;
    omk_batch *batch_ = nullptr;
    omk_tt *table_ = nullptr;
    int batch_capacity_ = 0;
    int last_n_ = 0;
    bool has_rave_ = false;
    std::vector<int32_t> h_paths_, h_len_, h_leaf_, h_actions_, h_roots_, h_moves_;
    void *d_moves_ = nullptr;  // recorded moves of the last selection that followed transpositions
    int64_t d_moves_ints_ = 0;
    std::array<int32_t, 5> redirect_counts_{0, 0, 0, 0, 0};
};

}  // namespace omk
