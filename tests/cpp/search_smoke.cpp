// Drives omk::GPUForestMCTSEngine<State> (csrc/omk_search.h) with a mock game state that has
// core::IGameState's method names, and omk::flattenTree with a mock node that has MCTSNode's
// accessors.  Prints what the Python test compares with the CPU checker.
//   search_smoke search <num_simulations> <batch_size> <widening 0|1> <noise 0|1> <temperature> [searches]
//     (searches > 1: that many searches one after the other on ONE engine, the last one printed)
//   search_smoke flatten
//
// The game: players 1 and 2 alternately take one of 12 cells; a player who takes a cell whose
// two ring neighbours are his wins; a full board is a draw.  The stand-in evaluator's value and
// policy are functions of the position only.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <vector>

#include "../../omoknuni_small_amd/csrc/omk_search.h"

enum class GameResult { ONGOING, WIN_PLAYER1, WIN_PLAYER2, DRAW };

class RingState {
   public:
    static constexpr int kCells = 12;
    std::unique_ptr<RingState> clone() const { return std::make_unique<RingState>(*this); }
    std::vector<int> getLegalMoves() const {
        std::vector<int> m;
        if (winner_ == 0)
            for (int i = 0; i < kCells; i++)
                if (cell_[i] == 0) m.push_back(i);
        return m;
    }
    void makeMove(int a) {
        cell_[a] = (char)player_;
        if (cell_[(a + 1) % kCells] == player_ && cell_[(a + kCells - 1) % kCells] == player_) winner_ = player_;
        player_ = 3 - player_;
        moves_++;
    }
    bool isTerminal() const { return winner_ != 0 || moves_ == kCells; }
    GameResult getGameResult() const {
        if (winner_ == 1) return GameResult::WIN_PLAYER1;
        if (winner_ == 2) return GameResult::WIN_PLAYER2;
        return moves_ == kCells ? GameResult::DRAW : GameResult::ONGOING;
    }
    int getCurrentPlayer() const { return player_; }
    int getActionSpaceSize() const { return kCells; }
    uint64_t getHash() const {
        uint64_t h = 1469598103934665603ull;
        for (int i = 0; i < kCells; i++) h = (h ^ (uint64_t)cell_[i]) * 1099511628211ull;
        return h ^ (uint64_t)player_;
    }

   private:
    char cell_[kCells] = {0};
    int player_ = 1, winner_ = 0, moves_ = 0;
};

// MCTSNode's accessors over a hand-made pointer tree
struct PtrNode {
    std::vector<std::shared_ptr<PtrNode>> children;
    int action = -1, visits = 0, vl = 0, rave_n = 0;
    float value_sum = 0.0f, prior = 0.0f, rave_sum = 0.0f;
    std::vector<std::shared_ptr<PtrNode>> &getChildren() { return children; }
    int getAction() const { return action; }
    int getVisitCount() const { return visits; }
    float getValue() const { return visits ? value_sum / visits : 0.0f; }
    float getPriorProbability() const { return prior; }
    int getVirtualLoss() const { return vl; }
    int getRAVECount() const { return rave_n; }
    float getRAVEValue() const { return rave_n ? rave_sum / rave_n : 0.0f; }
};

// the same with the two one-line accessors of the stored sums that flattenTree prefers when they exist
struct SumNode {
    std::vector<std::shared_ptr<SumNode>> children;
    int action = -1, visits = 0, rave_n = 0;
    float value_sum = 0.0f, prior = 0.0f, rave_sum = 0.0f;
    std::vector<std::shared_ptr<SumNode>> &getChildren() { return children; }
    int getAction() const { return action; }
    int getVisitCount() const { return visits; }
    float getValue() const { return visits ? value_sum / visits : 0.0f; }
    float getValueSum() const { return value_sum; }
    float getPriorProbability() const { return prior; }
    int getVirtualLoss() const { return 0; }
    int getRAVECount() const { return rave_n; }
    float getRAVEValue() const { return rave_n ? rave_sum / rave_n : 0.0f; }
    float getRAVEValueSum() const { return rave_sum; }
};

// stands for the reference's own mcts::NetworkOutput (include/mcts/evaluation_types.h:14-17): the search
// takes the evaluator's output type as it is
struct RefNetworkOutput {
    std::vector<float> policy;
    float value = 0.0f;
};

static int run_search(int sims, int batch, bool widening, bool noise, float temperature, int searches, bool follow) {
    omk::MCTSSettings s;
    s.num_simulations = sims;
    s.batch_size = batch;
    s.use_rave = false;
    s.use_progressive_widening = widening;
    s.add_dirichlet_noise = noise;
    s.temperature = temperature;
    s.max_depth = 16;
    s.transposition_table_size_mb = 1;  // 2^15 slots
    s.follow_transpositions = follow;
    using Engine = omk::GPUForestMCTSEngine<RingState, RefNetworkOutput>;
    long evaluated = 0;
    Engine::InferenceFunction evaluator = [&](const std::vector<std::unique_ptr<RingState>> &states) {
        std::vector<RefNetworkOutput> out(states.size());
        for (size_t i = 0; i < states.size(); i++) {
            const uint64_t h = states[i]->getHash();
            out[i].value = (float)((int)(h % 2001ull) - 1000) / 1000.0f;
            out[i].policy.resize(RingState::kCells);
            float sum = 0.0f;
            for (int a = 0; a < RingState::kCells; a++) {
                out[i].policy[(size_t)a] = (float)(1 + ((h >> (a * 3)) & 7ull));
                sum += out[i].policy[(size_t)a];
            }
            for (auto &p : out[i].policy) p /= sum;
        }
        evaluated += (long)states.size();
        return out;
    };
    Engine engine(evaluator, s, 200000);
    RingState root;
    root.makeMove(3);  // not the empty board: the root state has a history the leaves replay on top of
    omk::SearchResult r;
    for (int k = 0; k < searches; k++) {
        evaluated = 0;
        r = engine.search(root);  // every search starts a new tree: the table's entries for the old one are gone
    }
    printf("action %d value %.9g simulations %d nodes %lld evaluated %ld\n", r.action, r.value, r.simulations,
           (long long)r.nodes, evaluated);
    printf("table entries %lld transpositions %lld\n", (long long)r.table_entries, (long long)r.transpositions);
    printf("probabilities");
    for (float p : r.probabilities) printf(" %.9g", p);
    printf("\n");
    const int64_t n = engine.forest().nodeCount();
    std::vector<int32_t> N(n), VL(n), cb(n), cc(n), act(n);
    std::vector<float> W(n), P(n);
    omk_soa_view v;
    memset(&v, 0, sizeof(v));
    v.n_nodes = n;
    v.N = N.data();
    v.W = W.data();
    v.P = P.data();
    v.VL = VL.data();
    engine.forest().downloadStatistics(v);
    engine.forest().downloadStructure(n, cb.data(), cc.data(), act.data());
    for (int64_t i = 0; i < n; i++) printf("node %lld %d %.9g %.9g %d %d %d %d\n", (long long)i, N[i], W[i], P[i], VL[i], cb[i], cc[i], act[i]);
    // a terminal state is answered without a search
    RingState won;
    won.makeMove(0);
    won.makeMove(5);
    won.makeMove(2);
    won.makeMove(6);
    won.makeMove(1);  // player 1 holds 0, 1, 2
    omk::SearchResult t = engine.search(won);
    printf("terminal action %d value %.9g probabilities %zu\n", t.action, t.value, t.probabilities.size());
    return 0;
}

static int run_flatten() {
    // root -> {a (2 children), b (leaf), c (1 child)}
    auto mk = [](int action, int visits, float sum, float prior, int vl) {
        auto n = std::make_shared<PtrNode>();
        n->action = action;
        n->visits = visits;
        n->value_sum = sum;
        n->prior = prior;
        n->vl = vl;
        n->rave_n = visits / 2;
        n->rave_sum = sum / 4;
        return n;
    };
    PtrNode root;
    root.visits = 40;
    root.value_sum = 4.0f;
    auto a = mk(7, 20, 8.0f, 0.5f, 0), b = mk(2, 12, -3.0f, 0.3f, 3), c = mk(9, 7, 0.5f, 0.2f, 0);
    a->children = {mk(1, 9, 2.25f, 0.6f, 0), mk(4, 10, -5.0f, 0.4f, 0)};
    c->children = {mk(5, 6, 1.5f, 1.0f, 0)};
    root.children = {a, b, c};
    std::vector<PtrNode *> node_of_id;
    omk::FlatTree t = omk::flattenTree(root, &node_of_id);
    for (size_t i = 0; i < t.N.size(); i++)
        printf("flat %zu %d %.9g %.9g %d %d %.9g %d %d %d\n", i, t.N[i], t.W[i], t.P[i], t.VL[i], t.rN[i], t.rW[i],
               t.child_begin[i], t.child_count[i], t.action[i]);
    // value sums that (sum / visits) * visits does not give back in binary32: with the accessors of the stored
    // sums the arrays hold the sums themselves
    {
        SumNode sroot;
        sroot.visits = 100;
        int lossy = 0;
        for (int i = 0; i < 40; i++) {
            auto c = std::make_shared<SumNode>();
            c->action = i;
            c->visits = 3 + i;
            c->value_sum = 0.1f * (float)(i + 1) + 0.013f;
            c->rave_n = 7 + i;
            c->rave_sum = -0.37f * (float)(i + 1);
            c->prior = 0.025f;
            if (c->getValue() * (float)c->visits != c->value_sum) lossy++;
            sroot.children.push_back(c);
        }
        omk::FlatTree st = omk::flattenTree(sroot);
        int exact = 0;
        for (size_t i = 1; i < st.N.size(); i++)
            if (st.W[i] == sroot.children[i - 1]->value_sum && st.rW[i] == sroot.children[i - 1]->rave_sum) exact++;
        printf("sums exact %d of %zu, mean times visits differs from the sum for %d\n", exact, st.N.size() - 1, lossy);
    }
    // the flattened tree searches on the device
    omk::MCTSSettings s;
    s.max_depth = 4;
    s.use_rave = false;
    omk::ForestEngine engine([](const std::vector<omk::LeafItem> &l) { return std::vector<omk::NetworkOutput>(l.size()); }, s, 64);
    omk_soa_view v = t.view(false);
    engine.uploadTree(v);
    std::vector<omk::LeafItem> leaves;
    engine.selectLeafBatch(0, 6, leaves);
    for (const auto &lf : leaves) {
        printf("path");
        for (int id : lf.path) printf(" %d", id);
        printf(" moves");
        for (int m : lf.move_sequence) printf(" %d", m);
        printf("\n");
        if (node_of_id[(size_t)lf.node]->getAction() != (lf.move_sequence.empty() ? -1 : lf.move_sequence.back())) return 3;
    }
    return 0;
}

int main(int argc, char **argv) {
    try {
        if (argc >= 7 && !strcmp(argv[1], "search"))
            return run_search(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]) != 0, atoi(argv[5]) != 0, (float)atof(argv[6]),
                              argc >= 8 ? atoi(argv[7]) : 1, argc >= 9 && atoi(argv[8]) != 0);
        if (argc >= 2 && !strcmp(argv[1], "flatten")) return run_flatten();
    } catch (const std::exception &e) {
        fprintf(stderr, "search_smoke: %s\n", e.what());
        return 1;
    }
    return 2;
}
