// Drives omk::ForestEngine the way the reference's search loop drives its tree: a forest
// read from a flat binary file, a deterministic stand-in evaluator, a few batches.  Prints
// the statistics afterwards so that the Python test can compare them with the CPU checker.
//   engine_smoke <forest.bin> <num_simulations> <batch_size> <max_depth>
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
    try {
        omk::ForestEngine engine(evaluator, s, n);
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
        engine.downloadStatistics(v);
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
