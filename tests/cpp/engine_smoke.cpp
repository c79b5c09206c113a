// Drives omk::ForestEngine the way the reference's search loop drives its tree: a forest
// read from a flat binary file, a deterministic stand-in evaluator, a few batches.  Prints
// the statistics afterwards so that the Python test can compare them with the CPU checker.
//   engine_smoke <forest.bin> <num_simulations> <batch_size> <max_depth> [grow]
// With `grow` the leaves are expanded on the device (stand-in game rules: the legal moves
// and the policy are functions of the leaf and its move list) and the forest's size,
// structure and priors are printed too.
// forest.bin: int64 n, then N, W, P, VL, child_begin, child_count, action (n x 4 bytes each).
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../omoknuni_small_amd/csrc/omk_engine.h"

int main(int argc, char **argv) {
    if (argc < 5) return 2;
    FILE *fp = fopen(argv[1], "rb");
    if (!fp) return 2;
    int64_t n = 0;
    if (fread(&n, 8, 1, fp) != 1) return 2;
    std::vector<int32_t> N(n), VL(n), cb(n), cc(n), act(n);
    std::vector<float> W(n), P(n);
    auto rd = [&](void *p) { return fread(p, 4, (size_t)n, fp) == (size_t)n; };
    if (!rd(N.data()) || !rd(W.data()) || !rd(P.data()) || !rd(VL.data()) || !rd(cb.data()) || !rd(cc.data()) ||
        !rd(act.data()))
        return 2;
    fclose(fp);

    omk::MCTSSettings s;
    s.num_simulations = atoi(argv[2]);
    s.batch_size = atoi(argv[3]);
    s.max_depth = atoi(argv[4]);
    s.use_rave = false;
    s.use_progressive_widening = false;  // every legal move becomes a child: what the Python side restates
    long leaves_seen = 0;
    auto evaluator = [&](const std::vector<omk::LeafItem> &leaves) {
        std::vector<omk::NetworkOutput> out(leaves.size());
        for (size_t i = 0; i < leaves.size(); i++) {
            // a value that depends on the leaf and on the replayed move list
            int h = leaves[i].node * 31 + (int)leaves[i].move_sequence.size();
            for (int a : leaves[i].move_sequence) h = h * 17 + a;
            out[i].value = (float)((h % 2001 + 2001) % 2001 - 1000) / 1000.0f;
            if (leaves[i].path.size() != leaves[i].move_sequence.size() + 1 || leaves[i].path.back() != leaves[i].node)
                exit(3);
        }
        leaves_seen += (long)leaves.size();
        return out;
    };
    const bool grow = argc > 5;
    // the hash the stand-in evaluator and the stand-in rules share
    auto leaf_hash = [](const omk::LeafItem &lf) {
        int h = lf.node * 31 + (int)lf.move_sequence.size();
        for (int a : lf.move_sequence) h = h * 17 + a;
        return h;
    };
    const int action_space = 8;
    auto rules = [&](const std::vector<omk::LeafItem> &leaves) {
        std::vector<std::vector<int>> moves(leaves.size());
        for (size_t i = 0; i < leaves.size(); i++) {
            unsigned h = (unsigned)leaf_hash(leaves[i]);
            if (h % 7u == 0u) continue;  // terminal state
            int k = 1 + (int)(h % 4u);
            for (int a = 0; a < k; a++) moves[i].push_back((int)((h + 3u * (unsigned)a) % 10u));  // some lie outside
        }
        return moves;
    };
    try {
        omk::ForestEngine engine(
            [&](const std::vector<omk::LeafItem> &leaves) {
                std::vector<omk::NetworkOutput> out = evaluator(leaves);
                if (grow)
                    for (size_t i = 0; i < leaves.size(); i++) {
                        unsigned h = (unsigned)leaf_hash(leaves[i]);
                        out[i].policy.resize(action_space);
                        for (int a = 0; a < action_space; a++)
                            out[i].policy[a] = (float)((h + 5u * (unsigned)a) % 13u) / 10.0f - 0.1f;  // some outside [0,1]
                    }
                return out;
            },
            s, grow ? n + 100000 : n);
        if (grow) engine.setLegalMovesFunction(rules);
        omk_soa_view v = {};
        v.n_nodes = n;
        v.N = N.data();
        v.W = W.data();
        v.P = P.data();
        v.VL = VL.data();
        v.child_begin = cb.data();
        v.child_count = cc.data();
        v.action = act.data();
        engine.uploadTree(v);
        int done = engine.executeBatchedTreeSearch(0);
        if (!grow) engine.downloadStatistics(v);
        if (grow) {
            // the forest has grown: fetch everything at its new size
            const int64_t m = engine.nodeCount();
            N.assign(m, 0); VL.assign(m, 0); W.assign(m, 0.0f); P.assign(m, 0.0f);
            cb.assign(m, 0); cc.assign(m, 0); act.assign(m, 0);
            v.n_nodes = m;
            v.N = N.data(); v.W = W.data(); v.P = P.data(); v.VL = VL.data();
            engine.downloadStatistics(v);
            engine.downloadStructure(m, cb.data(), cc.data(), act.data());
            printf("done %d leaves %ld nodes %lld\n", done, leaves_seen, (long long)m);
            for (int64_t i = 0; i < m; i++)
                printf("%d %.9g %d %.9g %d %d %d\n", N[i], W[i], VL[i], P[i], cb[i], cc[i], act[i]);
            return 0;
        }
        printf("done %d leaves %ld\n", done, leaves_seen);
        for (int64_t i = 0; i < n; i++) printf("%d %.9g %d\n", N[i], W[i], VL[i]);
        // the error path: an exception, not a crash
        try {
            engine.backPropagateBatch(std::vector<float>(1, 0.0f));
            if (s.batch_size != 1) return 4;
        } catch (const std::runtime_error &) {
        }
    } catch (const std::exception &e) {
        fprintf(stderr, "engine error: %s\n", e.what());
        return 1;
    }
    return 0;
}
