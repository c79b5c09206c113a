// MCTSEngine::search over the device-resident forest, with the reference's own signatures.
//
// GPUForestMCTSEngine<State> is a template over the game state type; it uses exactly the methods of
// core::IGameState (reference include/core/igamestate.h:54-240) that the reference's search uses on
// this path: clone(), makeMove(), isTerminal(), getLegalMoves(), getActionSpaceSize(),
// getCurrentPlayer(), getGameResult().  Instantiated on core::IGameState it takes the engine's
// existing InferenceFunction unchanged:
//     std::function<std::vector<NetworkOutput>(const std::vector<std::unique_ptr<core::IGameState>>&)>
// (reference include/mcts/mcts_engine.h:230-231).  It follows MCTSEngine::search
// (src/mcts/mcts_engine_main.cpp:256-440) and runSearch / executeBatchedTreeSearch
// (src/mcts/mcts_engine_search.cpp:347-400, src/mcts/mcts_engine_batch_tree_simple.cpp:14-301):
// terminal state -> its value; else a one-node tree, the root expanded and evaluated, batches of
// select / leaf states / evaluate / expand / back up until num_simulations are done, then the move
// probabilities from the root's visit counts and the move drawn from them.  The leaf states are
// what the reference builds at :170-178: a clone of the root state with the path's moves replayed.
//
// flattenTree() turns a pointer tree with MCTSNode's accessors (reference
// include/mcts/mcts_node.h:88-110) into the arrays omk_forest_upload takes, so that a search the
// CPU engine began can go on on the device.
//
// Header-only; needs omk_engine.h (libomk_engine.so, libomk_forest.so).
#pragma once

#include <algorithm>
#include <cmath>
#include <deque>
#include <memory>
#include <numeric>
#include <random>
#include <type_traits>
#include <utility>

#include "omk_engine.h"

namespace omk {

// reference include/mcts/mcts_engine.h:199-211 (of the statistics block: what this path counts)
struct SearchResult {
    int action = -1;
    std::vector<float> probabilities;
    float value = 0.0f;
    int simulations = 0;
    int64_t nodes = 0;
    // the table of positions over the whole search (settings.use_transposition_table): entries stored,
    // and lookups that found ANOTHER visited node for the position reached: what the reference would
    // redirect to (src/mcts/mcts_engine_batch_tree_simple.cpp:141-157): counted, and followed only with
    // settings.follow_transpositions (then `transpositions` counts the redirects made)
    int64_t table_entries = 0, transpositions = 0;
};

// reference include/mcts/evaluation_types.h:49-73: a leaf waiting for the network, with the tree on the
// device: the node is an id, the path a list of ids
template <class State>
struct PendingEvaluation {
    int32_t node = -1;
    std::unique_ptr<State> state;
    std::vector<int32_t> path;
};

namespace detail {
// a state type that reports a position key (IGameState::getHash, include/core/igamestate.h)
template <class S, class = void>
struct has_hash : std::false_type {};
template <class S>
struct has_hash<S, std::void_t<decltype(std::declval<const S &>().getHash())>> : std::true_type {};
// a node type that reports its value sum and its RAVE value sum as they are stored (the reference's MCTSNode
// exposes the means only, include/mcts/mcts_node.h:93,163: one-line accessors a maintainer adds)
template <class N, class = void>
struct has_value_sum : std::false_type {};
template <class N>
struct has_value_sum<N, std::void_t<decltype(std::declval<const N &>().getValueSum())>> : std::true_type {};
template <class N, class = void>
struct has_rave_value_sum : std::false_type {};
template <class N>
struct has_rave_value_sum<N, std::void_t<decltype(std::declval<const N &>().getRAVEValueSum())>> : std::true_type {};
}  // namespace detail

// The arrays of a flattened tree, owning their memory; view() is what omk_forest_upload takes.
struct FlatTree {
    std::vector<int32_t> N, VL, rN, child_begin, child_count, action;
    std::vector<float> W, P, rW;
    omk_soa_view view(bool with_rave) {
        omk_soa_view v;
        v.n_nodes = (int64_t)N.size();
        v.N = N.data();
        v.W = W.data();
        v.P = P.data();
        v.VL = VL.data();
        v.rN = with_rave ? rN.data() : nullptr;
        v.rW = with_rave ? rW.data() : nullptr;
        v.child_begin = child_begin.data();
        v.child_count = child_count.data();
        v.action = action.data();
        v.legal = nullptr;
        v.hash = nullptr;
        return v;
    }
};

// Breadth-first flattening of a pointer tree: the root becomes node 0, the children of a node take
// consecutive ids in the order of its children vector (so "lowest child index wins a tie" keeps its
// meaning).  Node is anything with MCTSNode's accessors: getChildren() (a container of pointers to
// Node), getAction(), getVisitCount(), getValue(), getPriorProbability(), getVirtualLoss(),
// getRAVECount(), getRAVEValue().  The value sums: getValueSum() / getRAVEValueSum() when the node type
// has them (the stored sums: a search that goes on from the arrays is then bit for bit the one that
// would have gone on from the pointer tree); otherwise mean * visits, which in binary32 is NOT in
// general the sum the mean was divided from ((W / N) * N can differ from W in the last place), so
// statistics and near-tie selections of the continued search can differ from the pointer tree's.
// node_of_id (optional) receives the node behind every id.
template <class Node>
FlatTree flattenTree(Node &root, std::vector<Node *> *node_of_id = nullptr) {
    FlatTree t;
    std::vector<Node *> order;
    order.push_back(&root);
    for (size_t head = 0; head < order.size(); head++) {
        Node *node = order[head];
        auto &children = node->getChildren();
        t.child_begin.push_back(children.empty() ? 0 : (int32_t)order.size());
        t.child_count.push_back((int32_t)children.size());
        for (auto &c : children) order.push_back(&*c);
    }
    for (Node *node : order) {
        const int visits = node->getVisitCount();
        t.N.push_back(visits);
        if constexpr (detail::has_value_sum<Node>::value) t.W.push_back(node->getValueSum());
        else t.W.push_back(node->getValue() * (float)visits);
        t.P.push_back(node->getPriorProbability());
        t.VL.push_back(node->getVirtualLoss());
        const int rave_visits = node->getRAVECount();
        t.rN.push_back(rave_visits);
        if constexpr (detail::has_rave_value_sum<Node>::value) t.rW.push_back(node->getRAVEValueSum());
        else t.rW.push_back(node->getRAVEValue() * (float)rave_visits);
        t.action.push_back(node->getAction());
    }
    if (node_of_id) *node_of_id = order;
    return t;
}

// Output: what the inference function returns per state, anything with `policy` (std::vector<float>)
// and `value` (float) members: the reference's mcts::NetworkOutput passes through unchanged.
template <class State, class Output = NetworkOutput>
class GPUForestMCTSEngine {
   public:
    using StatePtr = std::unique_ptr<State>;
    // the reference's InferenceFunction (include/mcts/mcts_engine.h:230-231) with State = core::IGameState
    // and Output = mcts::NetworkOutput
    using InferenceFunction = std::function<std::vector<Output>(const std::vector<StatePtr> &)>;

    GPUForestMCTSEngine(InferenceFunction inference_fn, const MCTSSettings &settings, int64_t capacity_nodes,
                        int device = 0, uint64_t seed = 5489u)
        : inference_fn_(std::move(inference_fn)),
          engine_([](const std::vector<LeafItem> &) { return std::vector<NetworkOutput>(); }, settings, capacity_nodes,
                  device, false),
          random_engine_(seed),
          shuffle_engine_(seed + 1u) {}

    const MCTSSettings &getSettings() const { return engine_.settings(); }
    ForestEngine &forest() { return engine_; }

    // MCTSEngine::search (src/mcts/mcts_engine_main.cpp:256-440)
    SearchResult search(const State &state) {
        const MCTSSettings &st = engine_.settings();
        SearchResult result;
        const int action_space = state.getActionSpaceSize();
        if (state.isTerminal()) {  // :299-322
            const int res = (int)state.getGameResult();  // GameResult: ONGOING, WIN_PLAYER1, WIN_PLAYER2, DRAW
            const int player = state.getCurrentPlayer();
            if (res == 1) result.value = player == 1 ? 1.0f : -1.0f;
            else if (res == 2) result.value = player == 2 ? 1.0f : -1.0f;
            result.probabilities.assign((size_t)action_space, 0.0f);
            return result;
        }
        // a new tree of one node: the root (runSearch: createRootNode)
        int32_t zero_i = 0;
        float zero_f = 0.0f, one_f = 1.0f;
        int32_t act = -1;
        omk_soa_view v;
        v.n_nodes = 1;
        v.N = &zero_i;
        v.W = &zero_f;
        v.P = &one_f;
        v.VL = &zero_i;
        v.rN = nullptr;
        v.rW = nullptr;
        int32_t cb = 0, cc = 0;
        v.child_begin = &cb;
        v.child_count = &cc;
        v.action = &act;
        v.legal = nullptr;
        v.hash = nullptr;
        engine_.uploadTree(v);
        if constexpr (detail::has_hash<State>::value) {
            // the loop that follows transpositions goes by the nodes' own keys: the root's is the first
            if (engine_.followsTranspositions()) engine_.setPositionKeys({0}, {(uint64_t)state.getHash()});
        }

        std::vector<StatePtr> states;
        std::vector<float> values;
        int completed = 0;
        bool root_expanded = false;
        while (completed < st.num_simulations) {
            // the first batch is the root alone: it is expanded and evaluated before anything else
            // (runSearch: expandNonTerminalLeaf(root_)), and gets its Dirichlet noise
            const int n = root_expanded ? std::min(st.batch_size, st.num_simulations - completed) : 1;
            // phase 1 and the leaf gather: the leaf states are a clone of the root state with the path's
            // moves replayed (mcts_engine_batch_tree_simple.cpp:170-178)
            std::vector<PendingEvaluation<State>> pending = collectLeafBatch(state, n);
            states.clear();
            states.reserve(pending.size());
            for (auto &pe : pending) states.push_back(std::move(pe.state));
            bool follow = false;
            if constexpr (detail::has_hash<State>::value) follow = engine_.followsTranspositions();
            if (follow) {
                // the selection was the loop with the table itself (store, lookup, redirect)
                const std::array<int32_t, 5> c = engine_.lastRedirectCounts();
                result.table_entries += c[0];
                result.transpositions += c[3];
            }
            if constexpr (detail::has_hash<State>::value) {
                if (st.use_transposition_table && !follow) {
                    // the keys of the positions reached, from the game itself, then the table's part of the
                    // traversal (:116-162) over the paths just selected
                    key_nodes_.clear();
                    key_values_.clear();
                    for (size_t i = 0; i < pending.size(); i++) {
                        key_nodes_.push_back(pending[i].node);
                        key_values_.push_back((uint64_t)states[i]->getHash());
                    }
                    engine_.setPositionKeys(key_nodes_, key_values_);
                    const std::array<int32_t, 4> c = engine_.traverseTranspositionTable();
                    result.table_entries += c[0];
                    result.transpositions += c[3];
                }
            }
            std::vector<Output> raw = inference_fn_(states);  // phase 2 (:212-236)
            if (raw.size() != states.size()) throw std::runtime_error("inference function returned a short batch");
            std::vector<NetworkOutput> out(raw.size());
            for (size_t i = 0; i < raw.size(); i++) {
                out[i].policy = std::move(raw[i].policy);
                out[i].value = raw[i].value;
            }
            std::vector<std::vector<int>> legal(states.size());
            values.resize(out.size());
            for (size_t i = 0; i < states.size(); i++) {
                if (!states[i]->isTerminal()) legal[i] = states[i]->getLegalMoves();  // a terminal node stays a leaf
                // MCTSNode::expand shuffles the legal moves before it creates the children (reference
                // src/mcts/mcts_node.cpp:357-364), so that the children kept under progressive widening are
                // a random subset and not the moves of lowest index at every node of the tree
                if (st.shuffle_moves) shuffleMoves(legal[i]);
                values[i] = out[i].value;
            }
            engine_.expandLeafBatch(legal, out, action_space, follow ? &first_child_ : nullptr);  // phase 3, first half (:249-259)
            if constexpr (detail::has_hash<State>::value) {
                if (follow) keyNewChildren(states, legal);
            }
            if (!root_expanded) {
                root_expanded = true;
                if (st.add_dirichlet_noise) addDirichletNoise();
            }
            engine_.backPropagateBatch(values);  // (:276-281)
            completed += n;
        }
        result.simulations = completed;
        result.nodes = engine_.nodeCount();
        // the result (mcts_engine_main.cpp:365-440)
        result.probabilities = engine_.getActionProbabilities(0, st.temperature, action_space);
        if (!result.probabilities.empty()) {
            float sum = std::accumulate(result.probabilities.begin(), result.probabilities.end(), 0.0f);
            if (std::fabs(sum - 1.0f) > 0.1f && sum > 0.0f)
                for (auto &p : result.probabilities) p /= sum;
            if (st.temperature < 0.01f) {
                result.action = (int)std::distance(result.probabilities.begin(),
                                                   std::max_element(result.probabilities.begin(), result.probabilities.end()));
            } else {
                std::uniform_real_distribution<float> dist(0.0f, 1.0f);
                const float r = dist(random_engine_);
                float cumsum = 0.0f;
                for (size_t i = 0; i < result.probabilities.size(); i++) {
                    cumsum += result.probabilities[i];
                    if (r <= cumsum) {
                        result.action = (int)i;
                        break;
                    }
                }
            }
            if (result.action < 0)
                result.action = (int)std::distance(result.probabilities.begin(),
                                                   std::max_element(result.probabilities.begin(), result.probabilities.end()));
        }
        // the root's value
        int32_t n_root = 0;
        float w_root = 0.0f;
        rootStatistics(n_root, w_root);
        result.value = n_root > 0 ? w_root / (float)n_root : 0.0f;
        return result;
    }

    // Phase 1 and the leaf gather of one batch of n simulations from the root of the tree on the device:
    // what the reference's collectors hand to the evaluator (PendingEvaluation: node, state, path).
    std::vector<PendingEvaluation<State>> collectLeafBatch(const State &root_state, int n) {
        engine_.selectLeafBatch(0, n, leaves_);
        std::vector<PendingEvaluation<State>> pending(leaves_.size());
        for (size_t i = 0; i < leaves_.size(); i++) {
            StatePtr s = root_state.clone();
            for (int move : leaves_[i].move_sequence) s->makeMove(move);
            pending[i].node = leaves_[i].node;
            pending[i].state = std::move(s);
            pending[i].path = leaves_[i].path;
        }
        return pending;
    }

   private:
    // The loop that follows transpositions stores a child under the key of its position the first time the
    // child is selected (reference :116-128), and gets that key by replaying the moves on a clone of the root
    // state.  With the tree on the device the key has to be there before the selection: every child created by
    // this batch's expansions is keyed now, from the leaf state the host already holds (one clone + makeMove +
    // getHash per child).  The children of a leaf are the first of its move list, in that order; new ids are
    // handed out in simulation order, so a leaf's children end where the next expanded leaf's begin.
    void keyNewChildren(const std::vector<StatePtr> &states, const std::vector<std::vector<int>> &legal) {
        key_nodes_.clear();
        key_values_.clear();
        const int64_t n_after = engine_.nodeCount();
        for (size_t i = 0; i < states.size(); i++) {
            const int32_t first = first_child_[i];
            if (first < 0) continue;
            int64_t end = n_after;
            for (size_t j = 0; j < states.size(); j++)
                if (first_child_[j] > first && first_child_[j] < end) end = first_child_[j];
            for (int64_t c = first; c < end; c++) {
                StatePtr s = states[i]->clone();
                s->makeMove(legal[i][(size_t)(c - first)]);
                key_nodes_.push_back((int32_t)c);
                key_values_.push_back((uint64_t)s->getHash());
            }
        }
        if (!key_nodes_.empty()) engine_.setPositionKeys(key_nodes_, key_values_);
    }

    // Fisher-Yates from the last place down, one raw 32-bit output of the generator per place
    // (j = output mod (k + 1)): spelled out rather than std::shuffle, whose use of the generator is
    // the standard library's own, so that a test can restate it
    void shuffleMoves(std::vector<int> &moves) {
        for (size_t k = moves.size(); k-- > 1;) {
            const size_t j = (size_t)(shuffle_engine_() % (uint32_t)(k + 1));
            std::swap(moves[k], moves[j]);
        }
    }

    // MCTSEngine::addDirichletNoise (src/mcts/mcts_engine_eval.cpp:78-110): gamma(alpha, 1) samples from
    // the engine's own generator, one per child of the root
    void addDirichletNoise() {
        const int64_t n = engine_.nodeCount();
        std::vector<int32_t> cb((size_t)n), cc((size_t)n), act((size_t)n);
        engine_.downloadStructure(n, cb.data(), cc.data(), act.data());
        if (cc[0] <= 0) return;
        std::gamma_distribution<float> gamma(engine_.settings().dirichlet_alpha, 1.0f);
        std::vector<float> samples((size_t)cc[0]);
        for (auto &x : samples) x = gamma(random_engine_);
        engine_.addDirichletNoise(0, samples, engine_.settings().dirichlet_epsilon);
    }

    void rootStatistics(int32_t &n_root, float &w_root) {
        const int64_t n = engine_.nodeCount();
        std::vector<int32_t> N((size_t)n), VL((size_t)n);
        std::vector<float> W((size_t)n), P((size_t)n);
        omk_soa_view v;
        v.n_nodes = n;
        v.N = N.data();
        v.W = W.data();
        v.P = P.data();
        v.VL = VL.data();
        v.rN = nullptr;
        v.rW = nullptr;
        v.child_begin = v.child_count = v.action = nullptr;
        v.legal = nullptr;
        v.hash = nullptr;
        engine_.downloadStatistics(v);
        n_root = N[0];
        w_root = W[0];
    }

    InferenceFunction inference_fn_;
    ForestEngine engine_;
    std::mt19937 random_engine_;
    std::mt19937 shuffle_engine_;  // its own stream: noise and the move drawn do not depend on the tree's size
    std::vector<LeafItem> leaves_;
    std::vector<int32_t> key_nodes_, first_child_;
    std::vector<uint64_t> key_values_;
};

}  // namespace omk
