// Seeded synthetic search forests with the shapes and statistics of the benchmark
// configurations (host only, no GPU code).  A tree is grown the way a batched search
// grows it: rounds of `growth_width` PUCT descents with a temporary virtual loss (a reached
// leaf additionally repels the remaining descents of its round), every reached leaf above
// the depth limit is expanded, the temporary loss is cleared.  The
// statistics of a node are drawn once, independently, when its parent is expanded:
//   N  ~ min(Zipf(s), n_cap)           W ~ U[-N, N]           VL = 0
//   P  = softmax of N(0, sigma) logits over the legal children of the parent
//   an expanded node gets N = 1 + sum of its legal children's N, W redrawn in [-N, N]
//   RAVE: rN ~ min(Zipf(s), n_cap), rW ~ U[-rN, rN]
// The descent used for growing is this file's own float PUCT; it only decides the shape
// and is not a parity reference for anything.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

extern "C" {

typedef struct omk_synth_desc {
    int64_t n_trees;
    int64_t nodes_per_tree;
    int32_t dense;         // 1: every expanded node has `fanout` slots and a legal mask; 0: variable fan-out
    int32_t fanout;        // dense: slots per expanded node
    double legal_frac;     // dense: probability that a slot holds a child
    int32_t last_legal;    // dense: the last slot (pass) always holds a child
    double poisson_lambda; // variable: fan-out = clip(Poisson(lambda), fan_min, fan_max)
    int32_t fan_min;
    int32_t fan_max;
    double zipf_s;
    int32_t n_cap;
    double logit_sigma;
    int32_t max_depth;     // nodes at this depth are never expanded
    int32_t growth_width;  // descents per growth round
    int32_t has_rave;
    int32_t sort_by_prior; // store children in prior-descending order
    int32_t pw;            // growth descents only look at the first ceil(sqrt(N_parent)) children
    int32_t with_hash;
    float c_puct;
    int32_t virtual_loss;
    uint64_t seed;
} omk_synth_desc;

typedef struct omk_synth_out {
    int32_t *N;
    float *W;
    float *P;
    int32_t *VL;
    int32_t *rN;
    float *rW;
    int32_t *child_begin;
    int32_t *child_count;
    int32_t *action;
    uint32_t *legal;  // (n_total + 31) / 32 words, zero-initialised by the caller; NULL when !dense
    uint64_t *hash;
    int32_t *depth;   // optional
    int32_t *roots;   // n_trees
    int64_t *used;    // n_trees: node ids actually used in each tree
} omk_synth_out;

}  // extern "C"

namespace {

struct Rng {
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed) {}
    uint64_t next() {  // splitmix64
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double uniform() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }
    double normal() {
        double u1 = uniform(), u2 = uniform();
        if (u1 < 1e-300) u1 = 1e-300;
        return std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2);
    }
    int poisson(double lambda) {  // Knuth; lambda is small here
        double L = std::exp(-lambda), p = 1.0;
        int k = 0;
        do {
            k++;
            p *= uniform();
        } while (p > L);
        return k - 1;
    }
};

struct Zipf {
    std::vector<double> cdf;  // cdf[n-1] = P(X <= n), n < cap
    int cap;
    Zipf(double s, int cap_) : cap(cap_) {
        const int64_t M = 2000000;
        double zeta = 0.0;
        for (int64_t n = M; n >= 1; n--) zeta += std::pow((double)n, -s);
        zeta += std::pow((double)M, 1.0 - s) / (s - 1.0) - 0.5 * std::pow((double)M, -s);
        cdf.resize((size_t)std::max(cap - 1, 0));
        double acc = 0.0;
        for (int n = 1; n < cap; n++) {
            acc += std::pow((double)n, -s) / zeta;
            cdf[(size_t)n - 1] = acc;
        }
    }
    int sample(Rng &r) const {
        double u = r.uniform();
        auto it = std::lower_bound(cdf.begin(), cdf.end(), u);
        if (it == cdf.end()) return cap;
        return (int)(it - cdf.begin()) + 1;
    }
};

struct Tree {
    const omk_synth_desc &d;
    const omk_synth_out &o;
    const Zipf &zipf;
    int64_t base, cap, used;
    Rng rng;
    std::vector<int32_t> depth;   // local
    std::vector<int32_t> tmp_vl;  // local

    Tree(const omk_synth_desc &d_, const omk_synth_out &o_, const Zipf &z, int64_t tree)
        : d(d_), o(o_), zipf(z), base(tree * d_.nodes_per_tree), cap(d_.nodes_per_tree), used(0),
          rng(d_.seed * 0x9E3779B97F4A7C15ull + (uint64_t)tree * 0xD1B54A32D192ED03ull + 12345u),
          depth((size_t)d_.nodes_per_tree, 0), tmp_vl((size_t)d_.nodes_per_tree, 0) {}

    bool legal(int64_t g) const { return !o.legal || ((o.legal[g >> 5] >> (g & 31)) & 1u); }

    void draw_stats(int64_t g) {
        int n = zipf.sample(rng);
        o.N[g] = n;
        o.W[g] = (float)((rng.uniform() * 2.0 - 1.0) * n);
        o.VL[g] = 0;
        if (d.has_rave) {
            int rn = zipf.sample(rng);
            o.rN[g] = rn;
            o.rW[g] = (float)((rng.uniform() * 2.0 - 1.0) * rn);
        }
    }

    bool expand(int64_t local) {
        int f = d.dense ? d.fanout
                        : std::min(std::max(rng.poisson(d.poisson_lambda), (int)d.fan_min), (int)d.fan_max);
        if (used + f > cap) return false;
        const int64_t cb = used;
        used += f;
        std::vector<uint8_t> lg((size_t)f, 1);
        if (d.dense) {
            int any = 0;
            for (int i = 0; i < f; i++) {
                lg[(size_t)i] = rng.uniform() < d.legal_frac;
                any |= lg[(size_t)i];
            }
            if (d.last_legal) lg[(size_t)f - 1] = 1;
            else if (!any) lg[(size_t)(rng.next() % (uint64_t)f)] = 1;
        }
        std::vector<double> pr((size_t)f, 0.0);
        double mx = -1e300;
        for (int i = 0; i < f; i++)
            if (lg[(size_t)i]) {
                pr[(size_t)i] = rng.normal() * d.logit_sigma;
                mx = std::max(mx, pr[(size_t)i]);
            }
        double sum = 0.0;
        for (int i = 0; i < f; i++)
            if (lg[(size_t)i]) {
                pr[(size_t)i] = std::exp(pr[(size_t)i] - mx);
                sum += pr[(size_t)i];
            }
        std::vector<int> order((size_t)f);
        for (int i = 0; i < f; i++) order[(size_t)i] = i;
        if (d.sort_by_prior)
            std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return pr[(size_t)a] > pr[(size_t)b]; });
        int64_t nsum = 1;
        for (int k = 0; k < f; k++) {
            const int i = order[(size_t)k];
            const int64_t g = base + cb + k;
            o.child_begin[g] = 0;
            o.child_count[g] = 0;
            o.action[g] = i;
            depth[(size_t)(cb + k)] = depth[(size_t)local] + 1;
            if (o.depth) o.depth[g] = depth[(size_t)(cb + k)];
            if (lg[(size_t)i]) {
                if (o.legal) __atomic_fetch_or(&o.legal[g >> 5], 1u << (g & 31), __ATOMIC_RELAXED);
                draw_stats(g);
                o.P[g] = (float)(pr[(size_t)i] / sum);
                nsum += o.N[g];
            } else {
                o.N[g] = 0;
                o.W[g] = 0.0f;
                o.P[g] = 0.0f;
                o.VL[g] = 0;
                if (d.has_rave) {
                    o.rN[g] = 0;
                    o.rW[g] = 0.0f;
                }
            }
        }
        const int64_t gp = base + local;
        o.child_begin[gp] = (int32_t)(base + cb);
        o.child_count[gp] = f;
        o.N[gp] = (int32_t)std::min<int64_t>(nsum, 0x7FFFFFFF);
        o.W[gp] = (float)((rng.uniform() * 2.0 - 1.0) * (double)o.N[gp]);
        return true;
    }

    int64_t pick(int64_t local) {  // local index of the chosen child
        const int64_t gp = base + local;
        const int64_t cb = o.child_begin[gp] - base;
        int cc = o.child_count[gp];
        if (d.pw) {
            int k = (int)std::ceil(std::sqrt((double)o.N[gp]));
            cc = std::min(cc, std::max(k, 1));
        }
        const float ep = d.c_puct * std::sqrt((float)o.N[gp]);
        float best = -INFINITY;
        int64_t bi = -1;
        for (int i = 0; i < cc; i++) {
            const int64_t g = base + cb + i;
            if (!legal(g)) continue;
            const int vl = tmp_vl[(size_t)(cb + i)];
            const int ev = o.N[g] + vl;
            const float q = ev > 0 ? (o.W[g] - (float)vl) / (float)ev : 0.0f;
            const float s = q + o.P[g] * ep / (1.0f + (float)ev);
            if (s > best) {
                best = s;
                bi = cb + i;
            }
        }
        return bi;
    }

    void grow() {
        const int64_t groot = base;
        o.child_begin[groot] = 0;
        o.child_count[groot] = 0;
        o.action[groot] = -1;
        if (o.legal) __atomic_fetch_or(&o.legal[groot >> 5], 1u << (groot & 31), __ATOMIC_RELAXED);
        draw_stats(groot);
        o.P[groot] = 1.0f;
        if (o.depth) o.depth[groot] = 0;
        used = 1;
        if (!expand(0)) return;
        int64_t width = std::max(d.growth_width, 1);
        std::vector<int64_t> touched, queue;
        std::vector<uint8_t> queued((size_t)cap, 0);
        bool full = false;
        while (!full && width <= (1ll << 22)) {
            touched.clear();
            queue.clear();
            for (int64_t g = 0; g < width; g++) {
                int64_t node = 0;
                while (o.child_count[base + node] > 0) {
                    int64_t c = pick(node);
                    if (c < 0) break;
                    tmp_vl[(size_t)c] += d.virtual_loss;
                    touched.push_back(c);
                    node = c;
                }
                if (o.child_count[base + node] == 0 && depth[(size_t)node] < d.max_depth && !queued[(size_t)node]) {
                    queued[(size_t)node] = 1;
                    queue.push_back(node);
                }
                // a leaf that is already taken (or sits at the depth limit) repels the rest of
                // the round, so that every descent of a round ends somewhere new
                if (node != 0 && o.child_count[base + node] == 0) tmp_vl[(size_t)node] += 1 << 20;
            }
            for (int64_t c : touched) tmp_vl[(size_t)c] = 0;
            if (queue.empty()) {
                width *= 2;  // every reachable leaf sits at the depth limit: search wider
                continue;
            }
            for (int64_t node : queue)
                if (!expand(node)) {
                    full = true;
                    break;
                }
        }
    }
};

}  // namespace

extern "C" int omk_synth_generate(const omk_synth_desc *d, omk_synth_out *o) {
    if (!d || !o || d->n_trees <= 0 || d->nodes_per_tree < 2) return -1;
    if (d->n_trees * d->nodes_per_tree > 0x7FFFFFF0ll) return -1;
    if (d->dense && (d->fanout < 1 || d->fanout > 1024)) return -1;
    if (!d->dense && (d->fan_min < 1 || d->fan_max > 1024 || d->fan_min > d->fan_max)) return -1;
    if (!(d->zipf_s > 1.0) || d->n_cap < 1 || d->max_depth < 1) return -1;
    const Zipf zipf(d->zipf_s, d->n_cap);
    const int64_t total = d->n_trees * d->nodes_per_tree;
    // trees are independent; legal-mask words shared by neighbouring trees are set atomically
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t t = 0; t < d->n_trees; t++) {
        Tree tree(*d, *o, zipf, t);
        tree.grow();
        o->roots[t] = (int32_t)tree.base;
        if (o->used) o->used[t] = tree.used;
        // ids never handed out: childless, never referenced
        for (int64_t l = tree.used; l < tree.cap; l++) {
            const int64_t g = tree.base + l;
            o->N[g] = 0;
            o->W[g] = 0.0f;
            o->P[g] = 0.0f;
            o->VL[g] = 0;
            o->child_begin[g] = 0;
            o->child_count[g] = 0;
            o->action[g] = -1;
            if (d->has_rave) {
                o->rN[g] = 0;
                o->rW[g] = 0.0f;
            }
            if (o->depth) o->depth[g] = -1;
        }
    }
    if (d->with_hash && o->hash) {
#pragma omp parallel for schedule(static)
        for (int64_t g = 0; g < total; g++) {
            Rng r(d->seed ^ (0xA0761D6478BD642Full * (uint64_t)(g + 1)));
            uint64_t h = r.next();
            if (h == ~0ull) h = 0x1234567ull;
            o->hash[g] = h;
        }
    }
    return 0;
}
