// See omk_engine.h.  Plain host C++: links against libomk_forest.so, includes no HIP header.
#include "omk_engine.h"

#include <algorithm>

namespace omk {

ForestEngine::ForestEngine(InferenceFunction inference_fn, const MCTSSettings &settings, int64_t capacity_nodes,
                           int device, bool has_rave)
    : inference_fn_(std::move(inference_fn)), settings_(settings), has_rave_(has_rave) {
    omk_forest_desc desc;
    desc.capacity_nodes = capacity_nodes;
    desc.device = device;
    desc.has_rave = has_rave ? 1 : 0;
    check(omk_forest_create(&desc, &forest_), "omk_forest_create");
}

ForestEngine::~ForestEngine() {
    if (d_moves_) omk_dev_free(forest_, d_moves_);
    if (table_) omk_tt_destroy(table_);
    if (batch_) omk_batch_destroy(batch_);
    if (forest_) omk_forest_destroy(forest_);
}

void ForestEngine::check(int status, const char *what) const {
    if (status != OMK_OK) throw std::runtime_error(std::string(what) + ": " + omk_last_error());
}

void ForestEngine::uploadTree(const omk_soa_view &view) { check(omk_forest_upload(forest_, &view), "omk_forest_upload"); }

void ForestEngine::downloadStatistics(omk_soa_view &view) {
    check(omk_forest_download(forest_, &view), "omk_forest_download");
}

void ForestEngine::ensureBatch(int n) {
    if (batch_ && n <= batch_capacity_) return;
    if (batch_) {
        omk_batch_destroy(batch_);
        batch_ = nullptr;
    }
    batch_capacity_ = std::max(n, settings_.batch_size);
    check(omk_batch_create(forest_, batch_capacity_, settings_.max_depth, &batch_), "omk_batch_create");
}

void ForestEngine::selectLeafBatch(int32_t root, int batch_size, std::vector<LeafItem> &leaves) {
    h_roots_.assign((size_t)batch_size, root);
    selectLeafBatch(h_roots_, leaves);
}

void ForestEngine::selectLeafBatch(const std::vector<int32_t> &roots, std::vector<LeafItem> &leaves) {
    const int n = (int)roots.size();
    if (n <= 0) throw std::runtime_error("selectLeafBatch: empty batch");
    ensureBatch(n);
    check(omk_batch_set_roots(batch_, roots.data(), n), "omk_batch_set_roots");
    omk_select_params p;
    p.c_puct = settings_.exploration_constant;
    p.virtual_loss = settings_.virtual_loss;
    p.use_rave = (settings_.use_rave && has_rave_) ? 1 : 0;
    p.rave_k = settings_.rave_constant;
    p.pw = settings_.selection_prior_widening ? 1 : 0;
    const int D = settings_.max_depth;
    const bool follow = followsTranspositions();
    int stride = 0;
    if (follow) {
        ensureTable();
        omk_batch_dev dev;
        check(omk_batch_device(batch_, &dev), "omk_batch_device");
        stride = dev.stride;
        const int64_t want = (int64_t)D * stride;
        if (want > d_moves_ints_) {
            if (d_moves_) check(omk_dev_free(forest_, d_moves_), "omk_dev_free");
            d_moves_ = nullptr;
            check(omk_dev_alloc(forest_, want * 4, &d_moves_), "omk_dev_alloc");
            d_moves_ints_ = want;
        }
        check(omk_tt_select_redirect(table_, batch_, &p, (int32_t *)d_moves_, redirect_counts_.data()),
              "omk_tt_select_redirect");
    } else {
        check(omk_select_batch(batch_, &p), "omk_select_batch");
    }
    h_paths_.resize((size_t)n * (D + 1));
    h_len_.resize((size_t)n);
    h_leaf_.resize((size_t)n);
    h_actions_.resize((size_t)n * D);
    check(omk_batch_read(batch_, h_paths_.data(), h_len_.data(), h_leaf_.data(), h_actions_.data()), "omk_batch_read");
    if (follow) {
        // the recorded moves, level-major on the device: row d holds step d + 1 of every traversal
        h_moves_.resize((size_t)D * stride);
        check(omk_dev_d2h(forest_, h_moves_.data(), d_moves_, (int64_t)D * stride * 4), "omk_dev_d2h");
        for (int i = 0; i < n; i++)
            for (int d = 0; d + 1 < h_len_[(size_t)i]; d++)
                h_actions_[(size_t)i * D + d] = h_moves_[(size_t)d * stride + i];
    }
    leaves.clear();
    leaves.resize((size_t)n);
    for (int i = 0; i < n; i++) {
        LeafItem &it = leaves[(size_t)i];
        const int len = h_len_[(size_t)i];
        it.node = h_leaf_[(size_t)i];
        it.path.assign(h_paths_.begin() + (size_t)i * (D + 1), h_paths_.begin() + (size_t)i * (D + 1) + len);
        it.move_sequence.assign(h_actions_.begin() + (size_t)i * D, h_actions_.begin() + (size_t)i * D + (len - 1));
    }
    last_n_ = n;
}

void ForestEngine::backPropagateBatch(const std::vector<float> &leaf_values) {
    if ((int)leaf_values.size() != last_n_) throw std::runtime_error("backPropagateBatch: one value per selected leaf");
    check(omk_batch_set_values(batch_, leaf_values.data(), last_n_), "omk_batch_set_values");
    check(omk_backup_batch(batch_, settings_.virtual_loss), "omk_backup_batch");
}

std::vector<float> ForestEngine::getActionProbabilities(int32_t root, float temperature, int action_space) {
    std::vector<float> probs((size_t)action_space, 0.0f);
    int32_t children = 0;
    check(omk_forest_action_probabilities(forest_, root, temperature, action_space, probs.data(), &children),
          "omk_forest_action_probabilities");
    if (children == 0) probs.clear();  // the reference returns an empty vector for a root without children
    return probs;
}

void ForestEngine::addDirichletNoise(int32_t root, const std::vector<float> &gamma_samples, float epsilon) {
    check(omk_forest_add_root_noise(forest_, root, gamma_samples.data(), (int32_t)gamma_samples.size(), epsilon),
          "omk_forest_add_root_noise");
}

void ForestEngine::setPositionKeys(const std::vector<int32_t> &nodes, const std::vector<uint64_t> &keys) {
    if (nodes.size() != keys.size()) throw std::invalid_argument("setPositionKeys: one key per node");
    check(omk_forest_set_keys(forest_, nodes.data(), keys.data(), (int64_t)nodes.size()), "omk_forest_set_keys");
}

void ForestEngine::ensureTable() {
    if (table_) return;
    // 32 bytes per slot; the largest power of two that fits the configured size, 2^10 .. 2^26 slots
    int log2 = 10;
    while (log2 < 26 && (size_t(64) << log2) <= settings_.transposition_table_size_mb * (size_t(1) << 20)) log2++;
    check(omk_tt_create(forest_, log2, &table_), "omk_tt_create");
}

std::array<int32_t, 4> ForestEngine::traverseTranspositionTable() {
    ensureTable();
    std::array<int32_t, 4> counts{0, 0, 0, 0};
    check(omk_tt_traverse(table_, batch_, nullptr, 0, nullptr, nullptr, nullptr, nullptr, counts.data()), "omk_tt_traverse");
    return counts;
}

int64_t ForestEngine::nodeCount() const {
    int64_t n = 0;
    check(omk_forest_node_count(forest_, &n, nullptr), "omk_forest_node_count");
    return n;
}

void ForestEngine::downloadStructure(int64_t n_nodes, int32_t *child_begin, int32_t *child_count, int32_t *action) {
    check(omk_forest_download_structure(forest_, n_nodes, child_begin, child_count, action),
          "omk_forest_download_structure");
}

int64_t ForestEngine::expandLeafBatch(const std::vector<std::vector<int>> &legal_moves,
                                      const std::vector<NetworkOutput> &outputs, int action_space,
                                      std::vector<int32_t> *first_child) {
    if ((int)legal_moves.size() != last_n_) throw std::runtime_error("expandLeafBatch: one move list per simulation");
    const bool have_policy = outputs.size() == legal_moves.size();
    std::vector<int32_t> begin(legal_moves.size() + 1, 0), moves, pbegin(legal_moves.size() + 1, 0);
    std::vector<float> policy;
    for (size_t i = 0; i < legal_moves.size(); i++) {
        moves.insert(moves.end(), legal_moves[i].begin(), legal_moves[i].end());
        begin[i + 1] = (int32_t)moves.size();
        if (have_policy) {
            policy.insert(policy.end(), outputs[i].policy.begin(), outputs[i].policy.end());
            if (action_space <= 0 && !outputs[i].policy.empty()) action_space = (int)outputs[i].policy.size();
        }
        pbegin[i + 1] = (int32_t)policy.size();
    }
    if (moves.empty()) moves.push_back(0);
    const bool with_policy = have_policy && !policy.empty();
    omk_expand_params p;
    p.action_space = action_space;
    p.use_progressive_widening = settings_.use_progressive_widening ? 1 : 0;
    p.progressive_widening_c = settings_.progressive_widening_c;
    p.progressive_widening_k = settings_.progressive_widening_k;
    const int64_t before = nodeCount();
    if (first_child) first_child->assign(legal_moves.size(), -1);
    check(omk_expand_batch_ex(batch_, begin.data(), moves.data(), with_policy ? pbegin.data() : nullptr,
                              with_policy ? policy.data() : nullptr, &p, first_child ? first_child->data() : nullptr),
          "omk_expand_batch_ex");
    return nodeCount() - before;
}

int ForestEngine::executeBatchedTreeSearch(int32_t root) {
    int completed = 0;
    std::vector<LeafItem> leaves;
    std::vector<float> values;
    while (completed < settings_.num_simulations) {
        const int n = std::min(settings_.batch_size, settings_.num_simulations - completed);
        selectLeafBatch(root, n, leaves);
        std::vector<NetworkOutput> out = inference_fn_(leaves);
        if (out.size() != leaves.size()) throw std::runtime_error("inference function returned a short batch");
        values.resize(out.size());
        for (size_t i = 0; i < out.size(); i++) values[i] = out[i].value;
        if (legal_moves_fn_) expandLeafBatch(legal_moves_fn_(leaves), out);  // reference :249-259
        backPropagateBatch(values);
        completed += n;
    }
    check(omk_sync(forest_), "omk_sync");
    return completed;
}

}  // namespace omk
