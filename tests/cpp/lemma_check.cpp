// Brute-force check of keys_provably_monotone (csrc/omk_score.h) on the host: whenever the test
// says "provably monotone", every successive entry of the child, evaluated with the very
// arithmetic the kernels use, must not come before its predecessor.  Prints how often the test
// said yes; exits non-zero on the first counter-example.
//   g++ -O2 -std=c++17 -ffp-contract=off -fno-fast-math -I omoknuni_small_amd/csrc tests/cpp/lemma_check.cpp
#include <cstdio>
#include <cstdlib>
#include <random>

#include "omk_score.h"

using namespace omk;

template <bool RAVE>
static void entry(int n, float w, float p, int vl0, float q2, float ep, uint32_t uvl, int j, uint32_t &key,
                  uint32_t &pos) {
    const int vlj = (int)((uint32_t)vl0 + (uint32_t)j * uvl);
    uint32_t k1, k2;
    child_keys<RAVE>(n, w, p, vlj, q2, ep, k1, k2);
    if (k2 > k1) {
        key = k2;
        pos = 1;  // candidate of the second scan: after the first-scan candidate of the same child
    } else {
        key = k1;
        pos = 0;
    }
}

template <bool RAVE>
static long run(uint64_t seed, long cases, long *said_yes) {
    std::mt19937_64 g(seed);
    auto uni = [&](double a, double b) { return a + (b - a) * (double)(g() >> 11) / 9007199254740992.0; };
    long bad = 0;
    for (long c = 0; c < cases; c++) {
        const int shape = (int)(g() % 8);
        int n = 0;
        switch (shape) {
            case 0: n = 0; break;
            case 1: n = (int)(g() % 8); break;
            case 2: n = (int)(g() % 200); break;
            case 3: n = (int)(g() % 20000); break;
            default: n = (int)(g() % 12000000); break;
        }
        float w;
        switch ((int)(g() % 7)) {
            case 0: w = (float)-n; break;                                  // all losses
            case 1: w = (float)(-(double)n + uni(0, 2.0)); break;          // nearly all losses
            case 2: w = (float)n; break;
            case 3: w = (float)uni(-1.2 * n - 1, 1.2 * n + 1); break;      // also outside [-n, n]
            case 4: w = (float)((double)(long)uni(-n, n)); break;          // integral
            default: w = (float)uni(-(double)n, (double)n); break;
        }
        const float p = (g() % 11 == 0) ? 0.0f : (float)uni(0, 1.0) * (float)((g() % 5 == 0) ? 1e-4 : 1.0);
        const float ep = (float)(1.4 * sqrt(uni(0, 1) * uni(0, 1) * 2e6));
        const int vl0 = (g() % 3 == 0) ? (int)(g() % 50) : 0;
        const uint32_t uvl = 1u + (uint32_t)(g() % 4);
        const float q2 = (float)uni(-1.1, 1.1);
        const int j_last = 1 + (int)(g() % ((g() % 4 == 0) ? 20000 : 300));
        if (!keys_provably_monotone<RAVE>(n, w, p, vl0, q2, ep, uvl, j_last)) continue;
        (*said_yes)++;
        uint32_t pk, pp;
        entry<RAVE>(n, w, p, vl0, q2, ep, uvl, 0, pk, pp);
        if (pk == 0u) {
            bad++;
            printf("key 0 at visit 0: n %d w %.9g p %.9g vl0 %d ep %.9g\n", n, w, p, vl0, ep);
        }
        for (int j = 1; j <= j_last; j++) {
            uint32_t k, q;
            entry<RAVE>(n, w, p, vl0, q2, ep, uvl, j, k, q);
            if (k == 0u || k > pk || (k == pk && q < pp)) {
                bad++;
                printf("counter-example (rave %d): n %d w %.9g p %.9g vl0 %d q2 %.9g ep %.9g uvl %u visit %d: key %08x pos %u after "
                       "key %08x pos %u\n", (int)RAVE, n, w, p, vl0, q2, ep, uvl, j, k, q, pk, pp);
                break;
            }
            pk = k;
            pp = q;
        }
        if (bad > 5) break;
    }
    return bad;
}

int main(int argc, char **argv) {
    const long cases = argc > 1 ? atol(argv[1]) : 300000;
    long yes0 = 0, yes1 = 0;
    long bad = run<false>(12345, cases, &yes0) + run<true>(67890, cases, &yes1);
    printf("cases %ld per variant, provably monotone: %ld without RAVE, %ld with; counter-examples %ld\n", cases, yes0,
           yes1, bad);
    return bad ? 1 : 0;
}
