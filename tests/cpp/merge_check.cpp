// Host check of the rule by which the selection kernel settles a node where one child takes nearly
// every visitor (sparse_merge in csrc/omk_select.hip): the same steps, one "lane" at a time, with the
// score arithmetic of csrc/omk_score.h, on random nodes; every node the rule accepts is replayed
// one visitor at a time (the serial loop of the reference, mcts_engine_batch_tree_simple.cpp:73-185
// applied to one node) and must give the same winner order and the same visits per child.
// This pins the RULE (which children are listed, which child the others are merged into, the
// limit on a child's entries, the ranks, the refusals); the device code itself is held against the
// CPU checker by the GPU tests.
//   merge_check [cases [seed]]
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "omk_score.h"
using namespace omk;

static int F = 64;  // candidates of the second scan sit at positions F + child
static bool RAVE = true;
struct Kid {
    int n;
    float w, p;
    int vl;
    float q2;
    bool part;
    uint32_t k1, k2;
};
static void keys(const Kid &c, float ep, int vlj, uint32_t &k1, uint32_t &k2) {
    if (RAVE) child_keys<true>(c.n, c.w, c.p, vlj, c.q2, ep, k1, k2);
    else child_keys<false>(c.n, c.w, c.p, vlj, c.q2, ep, k1, k2);
}
static void entry_key(const Kid &c, float ep, uint32_t uvl, int j, int child, uint32_t &key, uint32_t &pos) {
    uint32_t k1, k2;
    keys(c, ep, (int)((uint32_t)c.vl + (uint32_t)j * uvl), k1, k2);
    if (k2 > k1) {
        key = k2;
        pos = (uint32_t)(F + child);
    } else {
        key = k1;
        pos = (uint32_t)child;
    }
}
static bool comes_before(uint32_t ka, uint32_t pa, uint32_t kb, uint32_t pb) { return ka > kb || (ka == kb && pa < pb); }
static float key_score(uint32_t key) {
    uint32_t b = (key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key;
    float f;
    memcpy(&f, &b, 4);
    return f;
}
// the closed-form estimate (approximate on purpose: it only seeds the exact search)
static int predict_count(const Kid &c, float ep, uint32_t uvl, float tau, int cap) {
    const float x0 = (float)c.n + (float)c.vl, A = c.w + (float)c.n, cc = c.p * ep, inv_step = 1.0f / (float)uvl;
    float xs = -1.0f;
    const float a2 = tau + 1.0f;
    if (a2 > 1e-12f) {
        const float b2 = a2 - A - cc, disc = b2 * b2 + 4.0f * a2 * A;
        if (disc >= 0.0f) xs = (-b2 + sqrtf(disc)) * (1.0f / (2.0f * a2));
    } else {
        xs = 3.0e38f;
    }
    if (RAVE) {
        const float d = tau - c.q2;
        xs = fmaxf(xs, d > 1e-12f ? cc * (1.0f / d) - 1.0f : 3.0e38f);
    }
    const float cnt = floorf((xs - x0) * inv_step) + 1.0f;
    if (!(cnt > 0.0f)) return 0;
    return cnt >= (float)cap ? cap : (int)cnt;
}
static int count_before(const Kid &c, float ep, uint32_t uvl, int child, uint32_t tk, uint32_t tp, int cap) {
    uint32_t kk, pp;
    auto before = [&](int j) {
        entry_key(c, ep, uvl, j, child, kk, pp);
        return kk != 0u && comes_before(kk, pp, tk, tp);
    };
    int lo = 1, hi = cap;  // entry 0 is known to come before (tk, tp)
    if (hi < lo) return lo;
    int g = predict_count(c, ep, uvl, key_score(tk), cap);
    g = g < lo ? lo : (g > hi ? hi : g);
    if (g > lo) {
        if (before(g - 1)) lo = g;
        else hi = g - 1;
    }
    if (lo == g && g < hi) {
        if (before(g)) lo = g + 1;
        else hi = g;
    }
    if (lo < hi) {
        const bool up = lo > g;
        for (int step = 2; lo < hi; step <<= 1) {
            int t = up ? lo + step : hi - step + 1;
            t = t > hi ? hi : (t <= lo ? lo + 1 : t);
            const bool b = before(t - 1);
            if (b) lo = t;
            else hi = t - 1;
            if (b != up) break;
        }
    }
    while (lo < hi) {
        const int t = (lo + hi + 1) >> 1;
        if (before(t - 1)) lo = t;
        else hi = t - 1;
    }
    return lo;
}

static int refusal = 0;
static bool sparse_merge(const std::vector<Kid> &k, float ep, uint32_t uvl, int m, int best0, uint32_t lk0, uint32_t lp0,
                         std::vector<uint32_t> &order, std::vector<int> &cnt) {
    const int nk = (int)k.size(), kSparseMax = 64;
    std::vector<int> L;  // the children that matter, in child order: one per lane
    for (int i = 0; i < nk; i++) {
        uint32_t hk = k[i].k1, hp = (uint32_t)i;
        if (k[i].k2 > k[i].k1) {
            hk = k[i].k2;
            hp = (uint32_t)(F + i);
        }
        if (hk != 0 && (i == best0 || comes_before(hk, hp, lk0, lp0))) L.push_back(i);
    }
    const int n0 = (int)L.size();
    if (n0 < 2 || n0 > kSparseMax) return refusal = 1, false;
    std::vector<uint32_t> hk(64, 0), hp(64, 0xFFFFFFFFu), zk(64, 0), zp(64, 0xFFFFFFFFu);
    for (int l = 0; l < n0; l++) {
        entry_key(k[L[l]], ep, uvl, 0, L[l], hk[l], hp[l]);
        entry_key(k[L[l]], ep, uvl, m - 1, L[l], zk[l], zp[l]);
    }
    uint32_t lk = 0, lp = 0xFFFFFFFFu;
    int a_lane = -1;
    for (int l = 0; l < n0; l++)
        if (zk[l] != 0 && comes_before(zk[l], zp[l], lk, lp)) {
            lk = zk[l];
            lp = zp[l];
            a_lane = l;
        }
    if (lk == 0) return refusal = 7, false;
    const Kid &A = k[L[a_lane]];
    const int a_child = L[a_lane];
    std::vector<bool> is_cand(64, false);
    bool any = false;
    for (int l = 0; l < n0; l++) {
        is_cand[l] = l != a_lane && hk[l] != 0 && comes_before(hk[l], hp[l], lk, lp);
        any = any || is_cand[l];
    }
    if (!any) return refusal = 9, false;
    int est_sum = 0;
    for (int l = 0; l < n0; l++)
        if (is_cand[l]) {
            const int r0 = predict_count(A, ep, uvl, key_score(hk[l]), m);
            const int room = m - r0 > 1 ? m - r0 : 1;
            est_sum += std::min(predict_count(k[L[l]], ep, uvl, key_score(lk), kSparseMax + 1), room);
        }
    if (est_sum > kSparseMax - 4) return refusal = 2, false;
    std::vector<unsigned long long> akp(m);
    {
        uint32_t pk = 0xFFFFFFFFu, ppos = 0;
        for (int j = 0; j < m; j++) {
            uint32_t kk, pp;
            entry_key(A, ep, uvl, j, a_child, kk, pp);
            akp[j] = ((unsigned long long)~kk << 32) | pp;
            if (kk == 0 || comes_before(kk, pp, pk, ppos)) return refusal = 5, false;
            pk = kk;
            ppos = pp;
        }
    }
    auto rank_in_a = [&](uint32_t tk, uint32_t tp) {
        const unsigned long long t64 = ((unsigned long long)~tk << 32) | tp;
        int lo = 0, hi = m;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (akp[mid] < t64) lo = mid + 1;
            else hi = mid;
        }
        return lo;
    };
    std::vector<int> cc(64, 0), cap(64, 1), start(64, 0);
    for (int l = 0; l < n0; l++)
        if (is_cand[l]) {
            int c = m - rank_in_a(hk[l], hp[l]);
            c = c > kSparseMax + 1 ? kSparseMax + 1 : (c < 1 ? 1 : c);
            cap[l] = c;
            cc[l] = count_before(k[L[l]], ep, uvl, L[l], lk, lp, c);
        }
    int total = 0;
    for (int l = 0; l < 64; l++) {
        start[l] = total;
        total += cc[l];
    }
    if (total > kSparseMax) return refusal = 3, false;
    std::vector<int> e_cl(64, -1), e_t(64, 0), rank_a(64, m), posn(64, 0);
    std::vector<uint32_t> ek(64, 0), epos(64, 0xFFFFFFFFu);
    for (int l = 0; l < 64; l++)
        for (int t = 0; t < cc[l]; t++) {
            e_cl[start[l] + t] = l;
            e_t[start[l] + t] = t;
        }
    int bad = 0;
    for (int e = 0; e < total; e++) {
        entry_key(k[L[e_cl[e]]], ep, uvl, e_t[e], L[e_cl[e]], ek[e], epos[e]);
        if (ek[e] == 0) bad = 1;
        rank_a[e] = rank_in_a(ek[e], epos[e]);
    }
    for (int e = 1; e < total; e++)
        if (e_t[e] > 0 && comes_before(ek[e], epos[e], ek[e - 1], epos[e - 1])) bad = std::max(bad, 2);
    std::vector<unsigned long long> e64(64, ~0ull);
    for (int e = 0; e < total; e++)
        e64[e] = ((unsigned long long)~ek[e] << 32) | ((unsigned long long)epos[e] << 8) | (unsigned)e;
    std::vector<bool> valid(64, false);
    for (int e = 0; e < total; e++) {
        int fr = 0;
        for (int o = 0; o < 64; o++) fr += e64[o] < e64[e] ? 1 : 0;
        posn[e] = rank_a[e] + fr;
        valid[e] = posn[e] < m;
    }
    for (int e = 1; e < total; e++)
        if (valid[e] && e_t[e] > 0 && !valid[e - 1]) bad = std::max(bad, 3);
    int nfv = 0;
    for (int e = 0; e < total; e++) nfv += valid[e];
    std::vector<int> mine_in(64, 0);
    for (int l = 0; l < n0; l++)
        if (is_cand[l]) {
            for (int t = 0; t < cc[l]; t++) mine_in[l] += valid[start[l] + t];
            if (mine_in[l] == cc[l] && cc[l] == cap[l]) bad = std::max(bad, 4);
        }
    if (bad) return refusal = 40 + bad, false;
    order.assign(m, 0);
    for (int e = 0; e < total; e++)
        if (valid[e]) order[posn[e]] = 0x80000000u | ((uint32_t)L[e_cl[e]] << 21) | (uint32_t)e_t[e];
    int seen = 0;
    for (int q = 0; q < m; q++) {
        if (order[q] >> 31) {
            order[q] &= 0x7FFFFFFFu;
            seen++;
        } else {
            order[q] = ((uint32_t)a_child << 21) | (uint32_t)(q - seen);
        }
    }
    if (seen != nfv) return refusal = 6, false;
    cnt.assign(nk, 0);
    for (int l = 0; l < n0; l++) cnt[L[l]] = l == a_lane ? m - nfv : mine_in[l];
    return true;
}

int main(int argc, char **argv) {
    const long cases = argc > 1 ? atol(argv[1]) : 100000;
    std::mt19937_64 rng(argc > 2 ? atoll(argv[2]) : 1);
    long merged = 0, wrong = 0, contested_n = 0, refusals[64] = {0};
    auto U = [&](double a, double b) { return std::uniform_real_distribution<double>(a, b)(rng); };
    for (long cs = 0; cs < cases; cs++) {
        RAVE = rng() & 1;
        const int nk = 2 + (int)(rng() % 40);
        const int m = 8 + (int)(rng() % (rng() % 3 == 0 ? 900 : 120));
        const uint32_t uvl = 1 + (uint32_t)(rng() % 4);
        const float ep = 1.4f * sqrtf((float)(100 + rng() % 100000));
        std::vector<Kid> k(nk);
        const int style = (int)(rng() % 4);
        for (int i = 0; i < nk; i++) {
            Kid &c = k[i];
            c.part = rng() % 10 != 0;
            c.n = style == 3 ? (int)(rng() % 3) : (int)(rng() % 60);
            if (rng() % 5 == 0) c.n = 0;
            c.w = (float)(U(-0.3, 0.6) * c.n);
            if (rng() % 7 == 0) c.w = floorf(c.w);
            c.p = (float)U(1e-5, style == 1 ? 0.05 : 0.005);
            c.vl = 0;
            const int rn = (int)(rng() % 40);
            c.q2 = RAVE ? combined_value(c.n, c.w, rn, (float)(U(-0.5, 0.5) * rn), 1000.0f) : 0.0f;
        }
        {  // a child that dominates
            Kid &c = k[rng() % nk];
            c.part = true;
            c.n = 1000 + (int)(rng() % 100000);
            c.w = (float)(U(0.7, 0.95) * c.n);
            c.p = (float)U(1e-4, 0.02);
            if (RAVE) c.q2 = combined_value(c.n, c.w, 500, (float)U(-200, 400), 1000.0f);
        }
        if (style == 2)  // rivals close to it
            for (int r = 0; r < 3; r++) {
                Kid &c = k[rng() % nk];
                c.part = true;
                c.n = 20 + (int)(rng() % 3000);
                c.w = (float)(U(0.6, 0.9) * c.n);
                c.p = (float)U(1e-4, 0.05);
                if (RAVE) c.q2 = combined_value(c.n, c.w, 300, (float)U(-100, 250), 1000.0f);
            }
        if (rng() % 6 == 0) {  // two children exactly alike: ties at every visit
            const int a = (int)(rng() % nk), b = (int)(rng() % nk);
            const bool pa = k[a].part;
            k[a] = k[b];
            k[a].part = pa || k[b].part;
        }
        for (auto &c : k) {
            c.k1 = c.k2 = 0;
            if (c.part) keys(c, ep, c.vl, c.k1, c.k2);
        }
        if (RAVE) {
            bool any1 = false;
            for (auto &c : k) any1 = any1 || c.k1 != 0;
            if (!any1)
                for (auto &c : k) c.k2 = 0;
        }
        // what the one-winner check finds first: the child with the best next entry, its entry for the
        // last visitor, the best next entry of the others
        int best = -1;
        uint32_t hk = 0, hp = 0xFFFFFFFFu, sk = 0, sp = 0xFFFFFFFFu;
        for (int i = 0; i < nk; i++)
            if (k[i].k1 > hk) hk = k[i].k1, hp = (uint32_t)i, best = i;
        for (int i = 0; i < nk; i++)
            if (k[i].k2 > hk) hk = k[i].k2, hp = (uint32_t)(F + i), best = i;
        if (best < 0) continue;
        for (int i = 0; i < nk; i++)
            if (i != best && k[i].k1 > sk) sk = k[i].k1, sp = (uint32_t)i;
        for (int i = 0; i < nk; i++)
            if (i != best && k[i].k2 > sk) sk = k[i].k2, sp = (uint32_t)(F + i);
        uint32_t lk0, lp0;
        entry_key(k[best], ep, uvl, m - 1, best, lk0, lp0);
        if (lk0 == 0 || !(sk != 0 && !comes_before(lk0, lp0, sk, sp))) continue;  // one winner, or no score
        contested_n++;
        std::vector<uint32_t> order;
        std::vector<int> cnt;
        refusal = 0;
        if (!sparse_merge(k, ep, uvl, m, best, lk0, lp0, order, cnt)) {
            refusals[refusal]++;
            continue;
        }
        merged++;
        std::vector<int> sc(nk, 0);  // the serial loop
        bool ok = true;
        for (int v = 0; v < m && ok; v++) {
            uint32_t bk = 0, bp = 0xFFFFFFFFu;
            int b = -1;
            for (int i = 0; i < nk; i++)
                if (k[i].part) {
                    uint32_t kk, pp;
                    entry_key(k[i], ep, uvl, sc[i], i, kk, pp);
                    if (kk != 0 && comes_before(kk, pp, bk, bp)) bk = kk, bp = pp, b = i;
                }
            if (b < 0 || order[v] != (((uint32_t)b << 21) | (uint32_t)sc[b])) ok = false;
            else sc[b]++;
        }
        int sum = 0;
        for (int i = 0; i < nk && ok; i++) {
            sum += cnt[i];
            if (cnt[i] != sc[i]) ok = false;
        }
        if (ok && sum != m) ok = false;
        if (!ok) {
            wrong++;
            if (wrong < 5) printf("WRONG: case %ld, rave %d, %d children, %d visitors, virtual loss %u\n", cs, (int)RAVE, nk, m, uvl);
        }
    }
    printf("nodes where the one-winner check fails: %ld; merged: %ld; wrong %ld; refused by reason:", contested_n, merged, wrong);
    for (int i = 0; i < 64; i++)
        if (refusals[i]) printf(" %d:%ld", i, refusals[i]);
    printf("\n");
    return wrong != 0;
}
