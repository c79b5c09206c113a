// C ABI of libomk_forest.so: handles, host<->device transfers, structural validation,
// and the launch glue of the selection / backup kernels.  Declarations and the reference
// interfaces they replace: include/omk_forest.h.
#include "../../include/omk_forest.h"

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "omk_internal.h"

using namespace omk;

static thread_local char g_err[512] = "";

static int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

#define HIP_TRY(expr)                                                                              \
    do {                                                                                           \
        hipError_t e_ = (expr);                                                                    \
        if (e_ != hipSuccess) return fail(OMK_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e_));    \
    } while (0)

struct omk_forest {
    int device = 0;
    int64_t capacity = 0;
    int64_t n_nodes = 0;
    bool has_rave = false;
    bool uploaded = false;
    bool prior_sorted = false;
    int max_fanout = 0;
    // Counts the changes that give node ids a new meaning (a compaction, an upload of a different
    // structure): paths, roots and work items of a batch made before such a change are stale.
    int64_t generation = 0;
    uint64_t structure_sum = 0;  // checksum of the child ranges last uploaded
    bool structure_changed = false;  // the device's child ranges are no longer the uploaded ones (expansion, compaction)
    hipStream_t own_stream = nullptr;
    hipStream_t stream = nullptr;
    // device arrays
    int2 *span = nullptr;
    int32_t *N = nullptr, *VL = nullptr, *rN = nullptr, *action = nullptr;
    float *W = nullptr, *P = nullptr, *rW = nullptr;
    // RAVE blend per node (ForestDev::q2): valid for the RAVE constant blend_k while blend_valid; whatever
    // changes N, W, rN or rW of nodes refreshes it or clears the flag
    float *Q2 = nullptr;
    bool blend_valid = false, blend_k_known = false;
    float blend_k = 0.0f;
    uint32_t *legal = nullptr;
    uint64_t *hash = nullptr;
    bool has_legal = false, has_action = false, has_hash = false;
    void *key_stage = nullptr;  // staging of omk_forest_set_keys: keys, node ids, one status word
    // Child slots re-pointed at transpositions (omk_tt_select_redirect): alias[s] >= 0 = the node slot s holds
    // instead of node s.  Allocated by the first such call; `redirected` once a slot has been re-pointed: the
    // forest is then a graph, and what assumes a tree refuses it until the next upload.
    int32_t *alias = nullptr;
    bool redirected = false;
    size_t key_stage_bytes = 0;
    int children = 0;       // live batches and tables created on this forest
    bool released = false;  // omk_forest_destroy was called while children were alive

    ForestMut mut() const {
        ForestMut m;
        m.span = span;
        m.N = N;
        m.W = W;
        m.P = P;
        m.VL = VL;
        m.rN = has_rave ? rN : nullptr;
        m.rW = has_rave ? rW : nullptr;
        m.q2 = has_rave ? Q2 : nullptr;
        m.legal = has_legal ? legal : nullptr;
        m.action = has_action ? action : nullptr;
        m.hash = has_hash ? hash : nullptr;
        return m;
    }

    ForestDev dev() const {
        ForestDev d;
        d.span = span;
        d.N = N;
        d.W = W;
        d.P = P;
        d.VL = VL;
        d.rN = has_rave ? rN : nullptr;
        d.rW = has_rave ? rW : nullptr;
        d.q2 = has_rave ? Q2 : nullptr;
        d.legal = has_legal ? legal : nullptr;
        d.action = has_action ? action : nullptr;
        d.hash = has_hash ? hash : nullptr;
        d.n_nodes = n_nodes;
        return d;
    }
};

constexpr int kSchedStep = 1024;  // int32 words between two scheduler words: 4 KiB
// Simulations cut by max_depth: two counters, used in turn (select calls of even / odd number).  Every
// select clears the counter of the next one, so that a select of lone traversals needs no reset launch.
constexpr int kTruncatedWord = 40;

struct omk_batch {
    omk_forest *f = nullptr;
    int32_t max_traversals = 0;
    int32_t max_depth = 0;
    int32_t stride = 0;
    int32_t n = 0;          // traversals bound by set_roots
    int64_t generation = -1;  // the forest's generation when the roots were set
    bool selected = false;  // paths of a select are on the device
    int32_t *paths = nullptr, *path_len = nullptr, *leaf = nullptr;
    float *values = nullptr;
    Item *items0 = nullptr, *items_q = nullptr, *singles0 = nullptr, *singles_q = nullptr;
    int32_t n_singles0 = 0;
    int32_t n_hctx0 = 0;  // contexts of heavy roots, handed out when the roots are set
    int32_t *seg0 = nullptr, *seg[2] = {nullptr, nullptr};
    int32_t *sc_child = nullptr, *sc_occ = nullptr;
    // [1..16] work statistics, [17] single-visitor queue length, [32] status of omk_batch_leaf_keys,
    // [40..41] simulations cut by max_depth (kTruncatedWord);
    // the scheduler words of the multi-visitor kernel follow at 4 KiB steps (kSchedStep), so
    // that each lies in a memory channel of its own
    int32_t *counters = nullptr;
    int32_t poll_sleep = 1;
    bool stats_on = false;
    bool trace_on = false;  // the selection records its timeline (omk_batch_set_trace)
    int32_t *q_ready = nullptr;  // per queue slot: number of the select call that published it
    int32_t *single_ready = nullptr;  // the same per entry of the single-visitor queue
    int32_t *hctx = nullptr;     // contexts of heavy nodes
    int32_t *hbound = nullptr;   // boundaries between their slices
    int32_t *list_flag = nullptr;  // per visitor-list start: which depth's list is complete
    int32_t hctx_cap = 0;
    int32_t q_cap = 0;
    int32_t epoch = 0;           // select calls so far
    int32_t spin_limit = 1 << 18;  // polls of about a microsecond: a quarter of a second, a selection takes a millisecond
    int32_t n_cus = 0;
    int32_t n_items0 = 0;
    int32_t *out_paths = nullptr, *out_actions = nullptr;  // row-major staging for the host
    int64_t out_ints = 0;  // int32 words of out_paths
    void *exp_buf = nullptr;  // staging of an expansion: jobs, moves, priors, status
    size_t exp_bytes = 0;
};

struct omk_tt {
    omk_forest *f = nullptr;
    int log2_slots = 0;
    TTSlot *slots = nullptr;
    TTMeta *meta = nullptr;
    int *d_status = nullptr;       // 8 counters of the last call
    uint32_t clock = 0;            // access_counter_ of the reference: entry i of a call has the time clock + i
    float threshold = 0.1f;        // Config::replacement_threshold
    void *work = nullptr;          // staging of store / traverse calls
    size_t work_bytes = 0;
    int64_t generation = -1;       // the forest's generation the stored node ids belong to (-1: nothing stored yet)
};

// The entries hold node ids.  They are the reference's weak_ptr entries, which die with the tree they
// point into (PHMapTranspositionTable::lookup erases an entry whose node is gone,
// src/mcts/phmap_transposition_table.cpp:100-108): once the forest's node ids have taken a new meaning
// (a compaction, an upload of another tree), every entry stored before is such a dead entry, and the
// table is emptied before anything else is done with it.  The access counter runs on, as the
// reference's does.
static int tt_same_tree(omk_tt *tt) {
    omk_forest *f = tt->f;
    if (tt->generation == f->generation) return OMK_OK;
    if (tt->generation >= 0) HIP_TRY(launch_tt_clear(tt->slots, tt->meta, tt->log2_slots, f->stream));
    tt->generation = f->generation;
    return OMK_OK;
}

static int tt_work(omk_tt *tt, size_t bytes) {
    if (bytes <= tt->work_bytes) return OMK_OK;
    HIP_TRY(hipStreamSynchronize(tt->f->stream));
    if (tt->work) HIP_TRY(hipFree(tt->work));
    tt->work = nullptr;
    tt->work_bytes = 0;
    HIP_TRY(hipMalloc(&tt->work, bytes));
    tt->work_bytes = bytes;
    return OMK_OK;
}

template <typename T>
static hipError_t dalloc(T **p, int64_t count) {
    return hipMalloc((void **)p, (size_t)std::max<int64_t>(count, 1) * sizeof(T));
}

static int use_device(const omk_forest *f) {
    if (f->released) return fail(OMK_ERR_STATE, "the forest of this handle has been destroyed");
    HIP_TRY(hipSetDevice(f->device));
    (void)hipGetLastError();  // launches are checked with hipGetLastError: start from a clean slate
    return OMK_OK;
}

// Roots, paths and work items of a batch are node ids: stale once the forest was compacted or a
// different structure uploaded.
static int tree_only(const char *who, const omk_forest *f) {
    if (f->redirected)
        return fail(OMK_ERR_UNSUPPORTED,
                    "%s: child slots of this forest have been re-pointed at transpositions (omk_tt_select_redirect): "
                    "it is a graph until the next upload, and this operation needs a tree", who);
    return OMK_OK;
}

static int fresh_batch(const char *who, const omk_batch *b) {
    if (b->generation != b->f->generation)
        return fail(OMK_ERR_STATE, "%s: the forest was compacted or uploaded with another structure since this "
                    "batch's roots were set; call omk_batch_set_roots and select again", who);
    return OMK_OK;
}

extern "C" {

const char *omk_last_error(void) { return g_err; }
int omk_version(void) { return 1; }

int omk_forest_create(const omk_forest_desc *desc, omk_forest **out) {
    if (!desc || !out) return fail(OMK_ERR_INVALID, "omk_forest_create: null argument");
    if (desc->capacity_nodes <= 0 || desc->capacity_nodes > 0x7FFFFFF0ll)
        return fail(OMK_ERR_INVALID, "omk_forest_create: capacity_nodes %lld out of range",
                    (long long)desc->capacity_nodes);
    int count = 0;
    HIP_TRY(hipGetDeviceCount(&count));
    if (desc->device < 0 || desc->device >= count)
        return fail(OMK_ERR_INVALID, "omk_forest_create: device %d of %d", desc->device, count);
    omk_forest *f = new (std::nothrow) omk_forest();
    if (!f) return fail(OMK_ERR_INVALID, "out of host memory");
    f->device = desc->device;
    f->capacity = desc->capacity_nodes;
    f->has_rave = desc->has_rave != 0;
    hipError_t e = hipSetDevice(f->device);
    if (e == hipSuccess) e = hipStreamCreate(&f->own_stream);
    const int64_t n = f->capacity;
    if (e == hipSuccess) e = dalloc(&f->span, n);
    if (e == hipSuccess) e = dalloc(&f->N, n);
    if (e == hipSuccess) e = dalloc(&f->W, n);
    if (e == hipSuccess) e = dalloc(&f->P, n);
    if (e == hipSuccess) e = dalloc(&f->VL, n);
    if (e == hipSuccess && f->has_rave) e = dalloc(&f->rN, n);
    if (e == hipSuccess && f->has_rave) e = dalloc(&f->rW, n);
    if (e == hipSuccess && f->has_rave) e = dalloc(&f->Q2, n);
    if (e != hipSuccess) {
        int rc = fail(OMK_ERR_HIP, "omk_forest_create: %s", hipGetErrorString(e));
        omk_forest_destroy(f);
        return rc;
    }
    f->stream = f->own_stream;
    *out = f;
    return OMK_OK;
}

static void forest_free(omk_forest *f) {
    (void)hipSetDevice(f->device);
    if (f->own_stream) (void)hipStreamSynchronize(f->own_stream);
    void *ptrs[] = {f->span, f->N, f->W, f->P, f->VL, f->rN, f->rW, f->Q2, f->action, f->legal, f->hash, f->key_stage, f->alias};
    for (void *p : ptrs)
        if (p) (void)hipFree(p);
    if (f->own_stream) (void)hipStreamDestroy(f->own_stream);
    (void)hipGetLastError();
    delete f;
}

// Batches and tables point into their forest: the memory goes when the last of them has.
static void forest_child_gone(omk_forest *f) {
    if (--f->children == 0 && f->released) forest_free(f);
}

int omk_forest_destroy(omk_forest *f) {
    if (!f) return OMK_OK;
    if (f->released) return fail(OMK_ERR_STATE, "omk_forest_destroy: called twice");
    if (f->children > 0) {
        f->released = true;
        return OMK_OK;
    }
    forest_free(f);
    return OMK_OK;
}

int omk_forest_set_stream(omk_forest *f, void *hip_stream) {
    if (!f) return fail(OMK_ERR_INVALID, "omk_forest_set_stream: null forest");
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipStreamSynchronize(f->stream));
    f->stream = hip_stream ? (hipStream_t)hip_stream : f->own_stream;
    return OMK_OK;
}

int omk_forest_get_stream(omk_forest *f, void **hip_stream_out) {
    if (!f || !hip_stream_out) return fail(OMK_ERR_INVALID, "omk_forest_get_stream: null argument");
    *hip_stream_out = (void *)f->stream;
    return OMK_OK;
}

int omk_sync(omk_forest *f) {
    if (!f) return fail(OMK_ERR_INVALID, "omk_sync: null forest");
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipStreamSynchronize(f->stream));
    return OMK_OK;
}

// The selection kernels give every node to exactly one wavefront per batch; that is only
// correct when every node is the child of at most one parent, so it is checked here, on
// the host, before anything reaches the device (it also keeps every child range in
// bounds, which is what protects the kernels from wild reads).
static int validate(const omk_soa_view *v, int64_t n, int *max_fanout, bool *prior_sorted, uint64_t *structure_sum) {
    std::vector<uint8_t> is_child((size_t)n, 0);
    int mf = 0;
    bool sorted = true;
    uint64_t h = 0xCBF29CE484222325ull ^ (uint64_t)n;  // checksum of (node, child range) of every expanded node
    for (int64_t i = 0; i < n; i++) {
        int32_t cc = v->child_count[i];
        if (cc == 0) continue;
        int32_t cb = v->child_begin[i];
        if (cc < 0) return fail(OMK_ERR_STRUCTURE, "node %lld: child_count %d < 0", (long long)i, cc);
        if (cc > OMK_MAX_FANOUT)
            return fail(OMK_ERR_STRUCTURE, "node %lld: child_count %d exceeds OMK_MAX_FANOUT %d", (long long)i, cc,
                        OMK_MAX_FANOUT);
        if (cb < 0 || (int64_t)cb + cc > n)
            return fail(OMK_ERR_STRUCTURE, "node %lld: children [%d, %d) outside [0, %lld)", (long long)i, cb,
                        cb + cc, (long long)n);
        for (int32_t c = cb; c < cb + cc; c++) {
            if (c == i) return fail(OMK_ERR_STRUCTURE, "node %lld is its own child", (long long)i);
            if (is_child[(size_t)c]) return fail(OMK_ERR_STRUCTURE, "node %d has two parents", c);
            is_child[(size_t)c] = 1;
            if (sorted && c > cb && !(v->P[c - 1] >= v->P[c])) sorted = false;
        }
        mf = std::max(mf, (int)cc);
        h = (h ^ ((uint64_t)i * 0x9E3779B97F4A7C15ull + ((uint64_t)(uint32_t)cb << 32) + (uint32_t)cc)) * 0x100000001B3ull;
    }
    *max_fanout = mf;
    *prior_sorted = sorted && v->legal == nullptr;
    *structure_sum = h;
    return OMK_OK;
}

int omk_forest_upload(omk_forest *f, const omk_soa_view *v) {
    if (!f || !v) return fail(OMK_ERR_INVALID, "omk_forest_upload: null argument");
    const int64_t n = v->n_nodes;
    if (n <= 0 || n > f->capacity)
        return fail(OMK_ERR_CAPACITY, "omk_forest_upload: %lld nodes, capacity %lld", (long long)n,
                    (long long)f->capacity);
    if (!v->N || !v->W || !v->P || !v->VL || !v->child_begin || !v->child_count)
        return fail(OMK_ERR_INVALID, "omk_forest_upload: N, W, P, VL, child_begin, child_count are required");
    if (f->has_rave && (!v->rN || !v->rW))
        return fail(OMK_ERR_INVALID, "omk_forest_upload: the forest was created with RAVE, rN and rW are required");
    int mf = 0;
    bool sorted = false;
    uint64_t ssum = 0;
    if (int rc = validate(v, n, &mf, &sorted, &ssum)) return rc;
    if (int rc = use_device(f)) return rc;

    std::vector<int2> span((size_t)n);
    for (int64_t i = 0; i < n; i++) {
        span[(size_t)i].x = v->child_begin[i];
        span[(size_t)i].y = v->child_count[i];
    }
    hipStream_t s = f->stream;
    HIP_TRY(hipStreamSynchronize(s));
    HIP_TRY(hipMemcpy(f->span, span.data(), (size_t)n * sizeof(int2), hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(f->N, v->N, (size_t)n * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(f->W, v->W, (size_t)n * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(f->P, v->P, (size_t)n * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(f->VL, v->VL, (size_t)n * 4, hipMemcpyHostToDevice));
    if (f->has_rave) {
        HIP_TRY(hipMemcpy(f->rN, v->rN, (size_t)n * 4, hipMemcpyHostToDevice));
        HIP_TRY(hipMemcpy(f->rW, v->rW, (size_t)n * 4, hipMemcpyHostToDevice));
    }
    f->has_action = v->action != nullptr;
    if (f->has_action) {
        if (!f->action) HIP_TRY(dalloc(&f->action, f->capacity));
        HIP_TRY(hipMemcpy(f->action, v->action, (size_t)n * 4, hipMemcpyHostToDevice));
    }
    f->has_legal = v->legal != nullptr;
    if (f->has_legal) {
        if (!f->legal) HIP_TRY(dalloc(&f->legal, (f->capacity + 31) / 32));
        HIP_TRY(hipMemcpy(f->legal, v->legal, (size_t)((n + 31) / 32) * 4, hipMemcpyHostToDevice));
    }
    f->has_hash = v->hash != nullptr;
    if (f->has_hash) {
        if (!f->hash) HIP_TRY(dalloc(&f->hash, f->capacity));
        HIP_TRY(hipMemcpy(f->hash, v->hash, (size_t)n * 8, hipMemcpyHostToDevice));
    }
    // the same structure again (statistics put back): node ids keep their meaning
    if (!f->uploaded || f->structure_changed || n != f->n_nodes || ssum != f->structure_sum) f->generation++;
    f->structure_sum = ssum;
    f->structure_changed = false;
    if (f->redirected) {  // an upload brings a tree: every slot holds its own node again
        HIP_TRY(launch_fill_words(f->alias, 0xFFFFFFFFu, f->capacity, f->stream));
        f->redirected = false;
    }
    f->n_nodes = n;
    f->max_fanout = mf;
    f->prior_sorted = sorted;
    f->uploaded = true;
    // the RAVE blend of every node from the new statistics, for the constant the selections have been using
    // (a first selection, or one with another constant, computes it itself)
    f->blend_valid = false;
    if (f->has_rave && f->blend_k_known) {
        HIP_TRY(launch_blend_all(f->dev(), f->blend_k, s));
        f->blend_valid = true;
    }
    return OMK_OK;
}

int omk_forest_download(omk_forest *f, omk_soa_view *v) {
    if (!f || !v) return fail(OMK_ERR_INVALID, "omk_forest_download: null argument");
    if (!f->uploaded) return fail(OMK_ERR_STATE, "omk_forest_download: nothing uploaded");
    if (v->n_nodes != f->n_nodes)
        return fail(OMK_ERR_INVALID, "omk_forest_download: view has %lld nodes, forest %lld", (long long)v->n_nodes,
                    (long long)f->n_nodes);
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipStreamSynchronize(f->stream));
    const size_t b = (size_t)f->n_nodes * 4;
    if (v->N) HIP_TRY(hipMemcpy(v->N, f->N, b, hipMemcpyDeviceToHost));
    if (v->W) HIP_TRY(hipMemcpy(v->W, f->W, b, hipMemcpyDeviceToHost));
    if (v->P) HIP_TRY(hipMemcpy(v->P, f->P, b, hipMemcpyDeviceToHost));
    if (v->VL) HIP_TRY(hipMemcpy(v->VL, f->VL, b, hipMemcpyDeviceToHost));
    if (f->has_rave && v->rN) HIP_TRY(hipMemcpy(v->rN, f->rN, b, hipMemcpyDeviceToHost));
    if (f->has_rave && v->rW) HIP_TRY(hipMemcpy(v->rW, f->rW, b, hipMemcpyDeviceToHost));
    return OMK_OK;
}

static inline bool view_legal(const omk_soa_view *v, int64_t i) {
    return !v->legal || ((v->legal[i >> 5] >> (i & 31)) & 1u);
}

int64_t omk_soa_count_legal(const omk_soa_view *v) {
    if (!v || v->n_nodes < 0) return fail(OMK_ERR_INVALID, "omk_soa_count_legal: null view");
    if (!v->legal) return v->n_nodes;
    int64_t c = 0;
    const int64_t words = v->n_nodes >> 5;
    for (int64_t w = 0; w < words; w++) c += __builtin_popcount(v->legal[w]);
    for (int64_t i = words << 5; i < v->n_nodes; i++) c += view_legal(v, i);
    return c;
}

int omk_soa_compact_legal(const omk_soa_view *v, int64_t count, int32_t *N, float *W, float *P, int32_t *VL,
                          int32_t *rN, float *rW, int32_t *child_begin, int32_t *child_count, int32_t *action,
                          uint64_t *hash, int32_t *old_to_new, int32_t *new_to_old) {
    if (!v || !N || !W || !P || !VL || !child_begin || !child_count)
        return fail(OMK_ERR_INVALID, "omk_soa_compact_legal: N, W, P, VL, child_begin, child_count are required");
    const int64_t n = v->n_nodes;
    if (n <= 0 || !v->N || !v->W || !v->P || !v->VL || !v->child_begin || !v->child_count)
        return fail(OMK_ERR_INVALID, "omk_soa_compact_legal: the view has no nodes or lacks a required array");
    if ((rN && !v->rN) || (rW && !v->rW) || (hash && !v->hash))
        return fail(OMK_ERR_INVALID, "omk_soa_compact_legal: rN, rW or hash asked for, the view has none");
    // rank[i]: kept nodes before node i
    std::vector<int32_t> rank((size_t)n + 1);
    int64_t c = 0;
    for (int64_t i = 0; i < n; i++) {
        rank[(size_t)i] = (int32_t)c;
        c += view_legal(v, i);
    }
    rank[(size_t)n] = (int32_t)c;
    if (c != count)
        return fail(OMK_ERR_INVALID, "omk_soa_compact_legal: the view keeps %lld nodes, room for %lld was announced",
                    (long long)c, (long long)count);
    if (action && !v->action)
        for (int64_t j = 0; j < c; j++) action[j] = -1;
    for (int64_t i = 0; i < n; i++) {
        if (old_to_new) old_to_new[i] = view_legal(v, i) ? rank[(size_t)i] : -1;
        if (!view_legal(v, i)) continue;
        const int64_t j = rank[(size_t)i];
        N[j] = v->N[i];
        W[j] = v->W[i];
        P[j] = v->P[i];
        VL[j] = v->VL[i];
        if (rN) rN[j] = v->rN[i];
        if (rW) rW[j] = v->rW[i];
        if (hash) hash[j] = v->hash[i];
        if (new_to_old) new_to_old[j] = (int32_t)i;
        const int64_t cb = v->child_begin[i], cc = v->child_count[i];
        if (cc < 0 || cb < 0 || cb + cc > n)
            return fail(OMK_ERR_INVALID, "omk_soa_compact_legal: node %lld has the child range [%lld, +%lld)", (long long)i,
                        (long long)cb, (long long)cc);
        child_count[j] = cc > 0 ? rank[(size_t)(cb + cc)] - rank[(size_t)cb] : 0;
        child_begin[j] = child_count[j] > 0 ? rank[(size_t)cb] : 0;
        if (action) {
            if (v->action) action[j] = v->action[i];
            else
                for (int64_t q = cb; q < cb + cc; q++)
                    if (view_legal(v, q)) action[rank[(size_t)q]] = (int32_t)(q - cb);
        }
    }
    return OMK_OK;
}

int omk_forest_download_structure(omk_forest *f, int64_t n_nodes, int32_t *h_child_begin, int32_t *h_child_count,
                                  int32_t *h_action) {
    if (!f) return fail(OMK_ERR_INVALID, "omk_forest_download_structure: null forest");
    if (!f->uploaded) return fail(OMK_ERR_STATE, "omk_forest_download_structure: nothing uploaded");
    if (n_nodes != f->n_nodes)
        return fail(OMK_ERR_INVALID, "omk_forest_download_structure: room for %lld nodes, forest has %lld",
                    (long long)n_nodes, (long long)f->n_nodes);
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipStreamSynchronize(f->stream));
    if (h_action) {
        if (f->has_action) {
            HIP_TRY(hipMemcpy(h_action, f->action, (size_t)n_nodes * 4, hipMemcpyDeviceToHost));
        } else {
            for (int64_t i = 0; i < n_nodes; i++) h_action[i] = (int32_t)i;
        }
    }
    if (h_child_begin || h_child_count) {
        std::vector<int2> sp((size_t)n_nodes);
        HIP_TRY(hipMemcpy(sp.data(), f->span, (size_t)n_nodes * sizeof(int2), hipMemcpyDeviceToHost));
        for (int64_t i = 0; i < n_nodes; i++) {
            if (h_child_begin) h_child_begin[i] = sp[(size_t)i].x;
            if (h_child_count) h_child_count[i] = sp[(size_t)i].y;
        }
    }
    return OMK_OK;
}

int omk_forest_set_keys(omk_forest *f, const int32_t *h_nodes, const uint64_t *h_keys, int64_t n) {
    if (!f || (n > 0 && (!h_nodes || !h_keys))) return fail(OMK_ERR_INVALID, "omk_forest_set_keys: null argument");
    if (!f->uploaded) return fail(OMK_ERR_STATE, "omk_forest_set_keys: nothing uploaded");
    if (n < 0) return fail(OMK_ERR_INVALID, "omk_forest_set_keys: n = %lld", (long long)n);
    if (int rc = use_device(f)) return rc;
    hipStream_t s = f->stream;
    if (!f->has_hash) {
        // a forest that came without position keys: every node starts with "no key"
        if (!f->hash) HIP_TRY(dalloc(&f->hash, f->capacity));
        HIP_TRY(launch_fill_words(f->hash, 0xFFFFFFFFu, f->capacity * 2, s));
        f->has_hash = true;
    }
    if (n == 0) return OMK_OK;
    // staging kept with the forest (a search calls this every batch): keys | node ids | status word
    const size_t need = (size_t)n * 12 + 8;
    if (need > f->key_stage_bytes) {
        HIP_TRY(hipStreamSynchronize(s));
        if (f->key_stage) HIP_TRY(hipFree(f->key_stage));
        f->key_stage = nullptr;
        f->key_stage_bytes = 0;
        const size_t room = need + need / 2;
        HIP_TRY(hipMalloc(&f->key_stage, room));
        f->key_stage_bytes = room;
    }
    uint64_t *d_keys = (uint64_t *)f->key_stage;
    int32_t *d_nodes = (int32_t *)(d_keys + n);
    int *d_bad = (int *)(d_nodes + n + (n & 1));
    int bad = 0;
    hipError_t e = hipMemcpyAsync(d_nodes, h_nodes, (size_t)n * 4, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipMemcpyAsync(d_keys, h_keys, (size_t)n * 8, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipMemcpyAsync(d_bad, &bad, 4, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = launch_set_keys(f->hash, d_nodes, d_keys, n, f->n_nodes, d_bad, s);
    if (e == hipSuccess) e = hipMemcpyAsync(&bad, d_bad, 4, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) return fail(OMK_ERR_HIP, "omk_forest_set_keys: %s", hipGetErrorString(e));
    if (bad) return fail(OMK_ERR_INVALID, "omk_forest_set_keys: %d node ids outside the forest (skipped)", bad);
    return OMK_OK;
}

int omk_forest_add_root_noise(omk_forest *f, int32_t root, const float *h_gamma, int32_t n_gamma, float epsilon) {
    if (!f || !h_gamma) return fail(OMK_ERR_INVALID, "omk_forest_add_root_noise: null argument");
    if (!f->uploaded) return fail(OMK_ERR_STATE, "omk_forest_add_root_noise: nothing uploaded");
    if (root < 0 || root >= f->n_nodes) return fail(OMK_ERR_INVALID, "omk_forest_add_root_noise: root %d", root);
    if (int rc = tree_only("omk_forest_add_root_noise", f)) return rc;
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipStreamSynchronize(f->stream));
    int2 sp;
    HIP_TRY(hipMemcpy(&sp, f->span + root, sizeof(sp), hipMemcpyDeviceToHost));
    const int32_t cb = sp.x, cc = sp.y;
    if (cc <= 0) return OMK_OK;  // no children to add noise to (mcts_engine_eval.cpp:78-80)
    std::vector<float> prior((size_t)cc);
    HIP_TRY(hipMemcpy(prior.data(), f->P + cb, (size_t)cc * 4, hipMemcpyDeviceToHost));
    std::vector<uint32_t> legal;
    const int64_t w0 = (int64_t)cb >> 5, w1 = ((int64_t)cb + cc + 31) >> 5;
    if (f->has_legal) {
        legal.resize((size_t)(w1 - w0));
        HIP_TRY(hipMemcpy(legal.data(), f->legal + w0, legal.size() * 4, hipMemcpyDeviceToHost));
    }
    auto is_child = [&](int32_t i) {
        if (!f->has_legal) return true;
        const int64_t id = (int64_t)cb + i;
        return ((legal[(size_t)((id >> 5) - w0)] >> (id & 31)) & 1u) != 0u;
    };
    int32_t children = 0;
    for (int32_t i = 0; i < cc; i++) children += is_child(i) ? 1 : 0;
    if (children == 0) return OMK_OK;
    if (n_gamma != children)
        return fail(OMK_ERR_INVALID, "omk_forest_add_root_noise: %d samples for %d children", n_gamma, children);
    // MCTSEngine::addDirichletNoise from the normalisation on, statement by statement
    float sum = 0.0f;
    for (int32_t j = 0; j < children; j++) sum = sum + h_gamma[j];
    std::vector<float> noise(h_gamma, h_gamma + children);
    if (sum > 0.0f) {
        for (auto &x : noise) x /= sum;
    } else {
        const float uniform_noise = 1.0f / (float)children;
        for (auto &x : noise) x = uniform_noise;
    }
    int32_t j = 0;
    for (int32_t i = 0; i < cc; i++) {
        if (!is_child(i)) continue;
        const float keep = (1.0f - epsilon) * prior[(size_t)i];
        const float add = epsilon * noise[(size_t)j++];
        prior[(size_t)i] = keep + add;
    }
    HIP_TRY(hipMemcpy(f->P + cb, prior.data(), (size_t)cc * 4, hipMemcpyHostToDevice));
    return OMK_OK;
}

int omk_forest_action_probabilities(omk_forest *f, int32_t root, float temperature, int32_t action_space,
                                    float *h_probabilities, int32_t *h_children) {
    if (!f || !h_probabilities) return fail(OMK_ERR_INVALID, "omk_forest_action_probabilities: null argument");
    if (!f->uploaded) return fail(OMK_ERR_STATE, "omk_forest_action_probabilities: nothing uploaded");
    if (root < 0 || root >= f->n_nodes || action_space <= 0)
        return fail(OMK_ERR_INVALID, "omk_forest_action_probabilities: root %d, action space %d", root, action_space);
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipStreamSynchronize(f->stream));
    int2 sp;
    HIP_TRY(hipMemcpy(&sp, f->span + root, sizeof(sp), hipMemcpyDeviceToHost));
    for (int32_t a = 0; a < action_space; a++) h_probabilities[a] = 0.0f;
    if (h_children) *h_children = 0;
    const int32_t cb = sp.x, cc = sp.y;
    if (cc <= 0) return OMK_OK;
    std::vector<int32_t> n((size_t)cc), act((size_t)cc);
    HIP_TRY(hipMemcpy(n.data(), f->N + cb, (size_t)cc * 4, hipMemcpyDeviceToHost));
    if (f->redirected) {
        // the counts are those of the nodes the children vector holds (child->getVisitCount(),
        // mcts_engine_tree.cpp:401-403), the actions those of the slots (root->getActions(), :395)
        std::vector<int32_t> al((size_t)cc);
        HIP_TRY(hipMemcpy(al.data(), f->alias + cb, (size_t)cc * 4, hipMemcpyDeviceToHost));
        for (int32_t i = 0; i < cc; i++)
            if (al[(size_t)i] >= 0) HIP_TRY(hipMemcpy(&n[(size_t)i], f->N + al[(size_t)i], 4, hipMemcpyDeviceToHost));
    }
    if (f->has_action) {
        HIP_TRY(hipMemcpy(act.data(), f->action + cb, (size_t)cc * 4, hipMemcpyDeviceToHost));
    } else {
        for (int32_t i = 0; i < cc; i++) act[(size_t)i] = cb + i;
    }
    std::vector<uint32_t> legal;
    const int64_t w0 = (int64_t)cb >> 5, w1 = ((int64_t)cb + cc + 31) >> 5;
    if (f->has_legal) {
        legal.resize((size_t)(w1 - w0));
        HIP_TRY(hipMemcpy(legal.data(), f->legal + w0, legal.size() * 4, hipMemcpyDeviceToHost));
    }
    auto is_child = [&](int32_t i) {
        if (!f->has_legal) return true;
        const int64_t id = (int64_t)cb + i;
        return ((legal[(size_t)((id >> 5) - w0)] >> (id & 31)) & 1u) != 0u;
    };
    // MCTSEngine::getActionProbabilities, statement by statement
    int32_t children = 0, max_idx = -1;
    float max_count = 0.0f;
    for (int32_t i = 0; i < cc; i++) {
        if (!is_child(i)) continue;
        children++;
        const float c = (float)n[(size_t)i];
        if (max_idx < 0 || c > max_count) {  // std::max_element: the first of the largest
            max_count = c;
            max_idx = i;
        }
    }
    if (h_children) *h_children = children;
    if (children == 0) return OMK_OK;
    const bool near_zero = temperature < 0.01f;
    float sum = 0.0f;
    if (!near_zero && max_count > 0.0f)
        for (int32_t i = 0; i < cc; i++) {
            if (!is_child(i)) continue;
            const float c = (float)n[(size_t)i];
            float scaled = 0.0f;
            if (c > 0.0f) scaled = powf(c / max_count, 1.0f / temperature);
            sum += scaled;
        }
    for (int32_t i = 0; i < cc; i++) {
        if (!is_child(i)) continue;
        float prob;
        if (near_zero) {
            prob = i == max_idx ? 1.0f : 0.0f;
        } else if (max_count <= 0.0f || !(sum > 0.0f)) {
            prob = 1.0f / (float)children;
        } else {
            const float c = (float)n[(size_t)i];
            float scaled = 0.0f;
            if (c > 0.0f) scaled = powf(c / max_count, 1.0f / temperature);
            prob = scaled / sum;
        }
        const int32_t a = act[(size_t)i];
        if (a >= 0 && a < action_space) h_probabilities[a] = prob;
    }
    return OMK_OK;
}

int omk_forest_reroot_child(omk_forest *f, int32_t root, int32_t last_action, int32_t *h_child) {
    if (!f || !h_child) return fail(OMK_ERR_INVALID, "omk_forest_reroot_child: null argument");
    if (!f->uploaded) return fail(OMK_ERR_STATE, "omk_forest_reroot_child: nothing uploaded");
    if (root < 0 || root >= f->n_nodes) return fail(OMK_ERR_INVALID, "omk_forest_reroot_child: root %d", root);
    *h_child = -1;
    if (last_action < 0) return OMK_OK;
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipStreamSynchronize(f->stream));
    int2 sp;
    HIP_TRY(hipMemcpy(&sp, f->span + root, sizeof(sp), hipMemcpyDeviceToHost));
    if (sp.y <= 0) return OMK_OK;
    std::vector<int32_t> act((size_t)sp.y);
    if (f->has_action) {
        HIP_TRY(hipMemcpy(act.data(), f->action + sp.x, (size_t)sp.y * 4, hipMemcpyDeviceToHost));
    } else {
        for (int32_t i = 0; i < sp.y; i++) act[(size_t)i] = sp.x + i;
    }
    std::vector<uint32_t> legal;
    const int64_t w0 = (int64_t)sp.x >> 5, w1 = ((int64_t)sp.x + sp.y + 31) >> 5;
    if (f->has_legal) {
        legal.resize((size_t)(w1 - w0));
        HIP_TRY(hipMemcpy(legal.data(), f->legal + w0, legal.size() * 4, hipMemcpyDeviceToHost));
    }
    for (int32_t i = 0; i < sp.y; i++) {
        const int64_t id = (int64_t)sp.x + i;
        if (f->has_legal && !((legal[(size_t)((id >> 5) - w0)] >> (id & 31)) & 1u)) continue;
        if (act[(size_t)i] == last_action) {
            *h_child = (int32_t)id;
            break;
        }
    }
    return OMK_OK;
}

// Device memory a compaction works in, beyond the forest's own arrays.
struct CompactScratch {
    int32_t *map = nullptr;    // [n] old id of every new node
    int32_t *begin = nullptr;  // [n] new id of every new node's first child
    int32_t *cc = nullptr;     // [n] child counts of the level at hand
    int32_t *scan = nullptr;   // [n] their exclusive prefix
    void *scan_tmp = nullptr;  // work space of the scan
    size_t scan_bytes = 0;
    uint64_t *tmp = nullptr;   // [n] the array every field passes through
    uint32_t *legal = nullptr; // [(n + 31) / 32] the new legal mask
};

// The compaction itself, in scratch memory the caller provides (room for the forest's node count).
static int compact_in(omk_forest *f, int32_t new_root, int64_t *h_nodes_after, int32_t *h_old_of_new,
                      const CompactScratch &sc) {
    hipStream_t s = f->stream;
    const int64_t n = f->n_nodes;
    // breadth-first order of the subtree, on the device: map[new id] = old id, begin[new id]
    // = new id of its first child.  One level per round; the levels' sizes come back to the
    // host (a handful of bytes per level).
    hipError_t e = hipMemcpyAsync(sc.map, &new_root, 4, hipMemcpyHostToDevice, s);
    int64_t lo = 0, hi = 1;
    bool not_a_tree = false;
    while (e == hipSuccess && hi > lo) {
        int64_t total = 0;
        e = launch_bfs_level(f->span, sc.map, sc.begin, lo, hi - lo, n - hi, sc.cc, sc.scan, sc.scan_tmp,
                             sc.scan_bytes, &total, s);
        if (e == hipSuccess && total > n - hi) {
            not_a_tree = true;
            break;
        }
        lo = hi;
        hi += total;
    }
    if (e != hipSuccess || not_a_tree) {
        (void)hipStreamSynchronize(s);
        if (not_a_tree) return fail(OMK_ERR_STRUCTURE, "omk_forest_compact: the child ranges do not form a tree");
        return fail(OMK_ERR_HIP, "omk_forest_compact: %s", hipGetErrorString(e));
    }
    const int64_t k = hi;
    auto move_words = [&](void *arr) {
        if (e != hipSuccess || !arr) return;
        e = launch_gather_words((uint32_t *)sc.tmp, (const uint32_t *)arr, sc.map, k, s);
        if (e == hipSuccess) e = launch_copy_words(arr, sc.tmp, k, s);
    };
    move_words(f->N);
    move_words(f->W);
    move_words(f->P);
    move_words(f->VL);
    if (f->has_rave) {
        move_words(f->rN);
        move_words(f->rW);
        move_words(f->Q2);  // the nodes keep their statistics, hence their RAVE blend
    }
    if (f->has_action) move_words(f->action);
    if (e == hipSuccess && f->has_hash) {
        e = launch_gather_dwords(sc.tmp, f->hash, sc.map, k, s);
        if (e == hipSuccess) e = launch_copy_words(f->hash, sc.tmp, k * 2, s);
    }
    if (e == hipSuccess) {
        e = launch_gather_span((int2 *)sc.tmp, f->span, sc.map, sc.begin, k, s);
        if (e == hipSuccess) e = launch_copy_words(f->span, sc.tmp, k * 2, s);
    }
    if (e == hipSuccess && f->has_legal) {
        e = launch_gather_legal(sc.legal, f->legal, sc.map, k, s);
        if (e == hipSuccess) e = launch_copy_words(f->legal, sc.legal, (k + 31) / 32, s);
    }
    if (e == hipSuccess && h_old_of_new) e = hipMemcpyAsync(h_old_of_new, sc.map, (size_t)k * 4, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) return fail(OMK_ERR_HIP, "omk_forest_compact: %s", hipGetErrorString(e));
    f->n_nodes = k;
    f->generation++;
    f->structure_changed = true;
    if (h_nodes_after) *h_nodes_after = k;
    return OMK_OK;
}

int omk_forest_compact(omk_forest *f, int32_t new_root, int64_t *h_nodes_after, int32_t *h_old_of_new) {
    if (!f) return fail(OMK_ERR_INVALID, "omk_forest_compact: null forest");
    if (!f->uploaded) return fail(OMK_ERR_STATE, "omk_forest_compact: nothing uploaded");
    if (new_root < 0 || new_root >= f->n_nodes) return fail(OMK_ERR_INVALID, "omk_forest_compact: root %d", new_root);
    if (int rc = tree_only("omk_forest_compact", f)) return rc;
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipStreamSynchronize(f->stream));
    const int64_t n = f->n_nodes;
    CompactScratch sc;
    hipError_t e = bfs_scan_bytes(n, &sc.scan_bytes);
    if (e == hipSuccess) e = hipMalloc((void **)&sc.map, (size_t)n * 4);
    if (e == hipSuccess) e = hipMalloc((void **)&sc.begin, (size_t)n * 4);
    if (e == hipSuccess) e = hipMalloc((void **)&sc.cc, (size_t)n * 4);
    if (e == hipSuccess) e = hipMalloc((void **)&sc.scan, (size_t)n * 4);
    if (e == hipSuccess) e = hipMalloc(&sc.scan_tmp, sc.scan_bytes > 0 ? sc.scan_bytes : 4);
    if (e == hipSuccess) e = hipMalloc((void **)&sc.tmp, (size_t)n * 8);
    if (e == hipSuccess && f->has_legal) e = hipMalloc((void **)&sc.legal, (size_t)((n + 31) / 32) * 4);
    int rc = e == hipSuccess ? compact_in(f, new_root, h_nodes_after, h_old_of_new, sc)
                             : fail(OMK_ERR_HIP, "omk_forest_compact: %s", hipGetErrorString(e));
    (void)hipStreamSynchronize(f->stream);
    for (void *p : {(void *)sc.map, (void *)sc.begin, (void *)sc.cc, (void *)sc.scan, (void *)sc.legal, (void *)sc.tmp,
                    sc.scan_tmp})
        if (p) (void)hipFree(p);
    return rc;
}

// ---- the same compaction for callers that cannot allocate ----
//
// All the scratch memory of a compaction of up to kStaticCompactNodes nodes, laid out in one
// file-scope device array: every GPU the library runs on holds its own copy for the life of the
// process.  In host code the array's name is only a handle for hipGetSymbolAddress; the address the
// kernels get is looked up once per device (static_scratch) and kept.
constexpr int64_t kStaticCompactNodes = 1ll << 20;
constexpr size_t kStaticScanBytes = 1u << 20;  // work space of the level scan (a few KiB are used)
constexpr size_t kStaticWords = (size_t)kStaticCompactNodes * 4;
constexpr size_t kStaticOffMap = 0;
constexpr size_t kStaticOffBegin = kStaticOffMap + kStaticWords;
constexpr size_t kStaticOffCc = kStaticOffBegin + kStaticWords;
constexpr size_t kStaticOffScan = kStaticOffCc + kStaticWords;
constexpr size_t kStaticOffTmp = kStaticOffScan + kStaticWords;
constexpr size_t kStaticOffLegal = kStaticOffTmp + 2 * kStaticWords;
constexpr size_t kStaticOffScanTmp = kStaticOffLegal + kStaticWords / 32;
constexpr size_t kStaticScratchBytes = kStaticOffScanTmp + kStaticScanBytes;
static_assert(kStaticOffScanTmp % 256 == 0 && kStaticOffLegal % 256 == 0, "parts of the scratch keep its alignment");

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static unsigned char *g_scratch_ptr[kMaxDevices];  // device address of `scratch` on every device, once known

// The device address of the scratch array on the forest's device (which must be current).
static int static_scratch(int device, unsigned char **out) {
    if (device < 0 || device >= kMaxDevices) return fail(OMK_ERR_INVALID, "device %d: at most %d devices", device, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void *p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(OMK_ERR_HIP, "hipGetSymbolAddress(scratch) on device %d: %s", device, hipGetErrorString(e));
        g_scratch_ptr[device] = (unsigned char *)p;
    }
    *out = g_scratch_ptr[device];
    return OMK_OK;
}

int omk_forest_compact_static(omk_forest *f, int32_t new_root, int64_t *h_nodes_after, int32_t *h_old_of_new) {
    if (!f) return fail(OMK_ERR_INVALID, "omk_forest_compact_static: null forest");
    if (!f->uploaded) return fail(OMK_ERR_STATE, "omk_forest_compact_static: nothing uploaded");
    if (new_root < 0 || new_root >= f->n_nodes)
        return fail(OMK_ERR_INVALID, "omk_forest_compact_static: root %d", new_root);
    if (int rc = tree_only("omk_forest_compact_static", f)) return rc;
    if (f->n_nodes > kStaticCompactNodes)
        return fail(OMK_ERR_CAPACITY,
                    "omk_forest_compact_static: the forest holds %lld nodes, the static scratch memory serves at most "
                    "%lld; use omk_forest_compact",
                    (long long)f->n_nodes, (long long)kStaticCompactNodes);
    if (int rc = use_device(f)) return rc;
    unsigned char *base = nullptr;
    if (int rc = static_scratch(f->device, &base)) return rc;
    HIP_TRY(hipStreamSynchronize(f->stream));
    CompactScratch sc;
    size_t need = 0;
    HIP_TRY(bfs_scan_bytes(f->n_nodes, &need));
    if (need > kStaticScanBytes)
        return fail(OMK_ERR_CAPACITY, "omk_forest_compact_static: the level scan wants %zu bytes of work space, %zu are reserved",
                    need, kStaticScanBytes);
    // every part is written by this call before it is read (the order map from the root on, the
    // counts and their scan per level, the staging array per field): nothing has to start at zero
    sc.map = (int32_t *)(base + kStaticOffMap);
    sc.begin = (int32_t *)(base + kStaticOffBegin);
    sc.cc = (int32_t *)(base + kStaticOffCc);
    sc.scan = (int32_t *)(base + kStaticOffScan);
    sc.tmp = (uint64_t *)(base + kStaticOffTmp);
    sc.legal = (uint32_t *)(base + kStaticOffLegal);
    sc.scan_tmp = base + kStaticOffScanTmp;
    sc.scan_bytes = kStaticScanBytes;
    return compact_in(f, new_root, h_nodes_after, h_old_of_new, sc);
}

int omk_forest_node_count(omk_forest *f, int64_t *h_nodes, int64_t *h_capacity) {
    if (!f) return fail(OMK_ERR_INVALID, "omk_forest_node_count: null forest");
    if (h_nodes) *h_nodes = f->n_nodes;
    if (h_capacity) *h_capacity = f->capacity;
    return OMK_OK;
}

// ---------------------------------------------------------------- batch

int omk_batch_create(omk_forest *f, int32_t max_traversals, int32_t max_depth, omk_batch **out) {
    if (!f || !out) return fail(OMK_ERR_INVALID, "omk_batch_create: null argument");
    if (max_traversals <= 0 || max_traversals > (1 << 24))
        return fail(OMK_ERR_INVALID, "omk_batch_create: max_traversals %d out of range", max_traversals);
    if (max_depth <= 0 || max_depth > 4096)
        return fail(OMK_ERR_INVALID, "omk_batch_create: max_depth %d out of range", max_depth);
    if ((int64_t)max_traversals * (max_depth + 1) > (1ll << 28))
        return fail(OMK_ERR_CAPACITY, "omk_batch_create: max_traversals x (max_depth+1) = %lld exceeds 2^28",
                    (long long)max_traversals * (max_depth + 1));
    if (int rc = use_device(f)) return rc;
    omk_batch *b = new (std::nothrow) omk_batch();
    if (!b) return fail(OMK_ERR_INVALID, "out of host memory");
    b->f = f;
    f->children++;
    b->max_traversals = max_traversals;
    b->max_depth = max_depth;
    b->stride = (max_traversals + 63) & ~63;
    const int64_t B = b->stride;
    hipError_t e = dalloc(&b->paths, B * (max_depth + 1));
    if (e == hipSuccess) e = dalloc(&b->path_len, B);
    if (e == hipSuccess) e = dalloc(&b->leaf, B);
    if (e == hipSuccess) e = dalloc(&b->values, B);
    if (e == hipSuccess) e = dalloc(&b->items0, B);
    // a multi-visitor item has at least two visitors, and a level holds each visitor once; a heavy
    // node (kHeavyMin visitors or more) adds at most 63 slice items
    // (and as many parts of its partition, and as many boundaries worked out ahead of time)
    b->q_cap = (int32_t)((B + 64) * (max_depth + 1));
    // (a node whose boundaries are worked out ahead of time, and that is then not cut into slices after all, uses
    // a second context for its partition)
    b->hctx_cap = (int32_t)std::min<int64_t>(4096, 2 * (B / kHeavyMin) * (max_depth + 1));
    if (e == hipSuccess) e = dalloc(&b->hctx, (int64_t)b->hctx_cap * kHeavyCtxInts);
    // (a context says by the number of the select call that its children's contexts are listed: memory that an
    // earlier batch left behind would say so for this batch's first calls, whose numbers start again at 1)
    if (e == hipSuccess)
        e = hipMemset(b->hctx, 0, (size_t)std::max<int64_t>((int64_t)b->hctx_cap * kHeavyCtxInts, 1) * 4);
    if (e == hipSuccess) e = dalloc(&b->hbound, (int64_t)b->hctx_cap * kMaxSlices * kBoundInts);
    if (e == hipSuccess)
        e = hipMemset(b->hbound, 0, (size_t)std::max<int64_t>((int64_t)b->hctx_cap * kMaxSlices * kBoundInts, 1) * 4);
    if (e == hipSuccess) e = dalloc(&b->list_flag, B);
    if (e == hipSuccess) e = dalloc(&b->items_q, b->q_cap);
    if (e == hipSuccess) e = dalloc(&b->q_ready, b->q_cap);
    if (e == hipSuccess) e = hipMemset(b->q_ready, 0, (size_t)std::max(b->q_cap, 1) * 4);
    if (e == hipSuccess) e = dalloc(&b->singles0, B);
    if (e == hipSuccess) e = dalloc(&b->singles_q, B);
    if (e == hipSuccess) e = dalloc(&b->seg0, B);
    if (e == hipSuccess) e = dalloc(&b->seg[0], B);
    if (e == hipSuccess) e = dalloc(&b->seg[1], B);
    if (e == hipSuccess) e = dalloc(&b->sc_child, 2 * B);  // two halves, alternating with the depth
    if (e == hipSuccess) e = dalloc(&b->sc_occ, 2 * B);
    if (e == hipSuccess) e = dalloc(&b->counters, 5 * kSchedStep);
    if (e == hipSuccess) e = hipMemset(b->counters, 0, 5 * kSchedStep * 4);
    if (e == hipSuccess) e = dalloc(&b->single_ready, max_traversals);
    if (e == hipSuccess) e = hipMemset(b->single_ready, 0, (size_t)std::max(max_traversals, 1) * 4);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&b->n_cus, hipDeviceAttributeMultiprocessorCount, f->device);
    // (also the staging of the timeline records, omk_debug_trace: room for 16384 of them at least)
    b->out_ints = std::max<int64_t>(B * (max_depth + 1), 24 * 16384);
    if (e == hipSuccess) e = dalloc(&b->out_paths, b->out_ints);
    if (e == hipSuccess) e = dalloc(&b->out_actions, B * max_depth);
    if (e == hipSuccess) e = hipMemset(b->values, 0, (size_t)B * 4);
    if (e != hipSuccess) {
        int rc = fail(OMK_ERR_HIP, "omk_batch_create: %s", hipGetErrorString(e));
        omk_batch_destroy(b);
        return rc;
    }
    *out = b;
    return OMK_OK;
}

int omk_batch_destroy(omk_batch *b) {
    if (!b) return OMK_OK;
    (void)hipSetDevice(b->f->device);
    (void)hipStreamSynchronize(b->f->stream);
    void *ptrs[] = {b->paths,  b->path_len, b->leaf,     b->values, b->items0,   b->items_q,  b->seg0,
                    b->seg[0], b->seg[1],   b->sc_child, b->sc_occ, b->counters, b->out_paths, b->out_actions,
                    b->singles0, b->singles_q, b->q_ready, b->hctx, b->hbound, b->exp_buf, b->list_flag, b->single_ready};
    for (void *p : ptrs)
        if (p) (void)hipFree(p);
    (void)hipGetLastError();
    forest_child_gone(b->f);
    delete b;
    return OMK_OK;
}

int omk_batch_set_roots(omk_batch *b, const int32_t *h_roots, int32_t n) {
    if (!b || !h_roots) return fail(OMK_ERR_INVALID, "omk_batch_set_roots: null argument");
    if (n <= 0 || n > b->max_traversals)
        return fail(OMK_ERR_CAPACITY, "omk_batch_set_roots: %d traversals, batch holds %d", n, b->max_traversals);
    omk_forest *f = b->f;
    if (!f->uploaded) return fail(OMK_ERR_STATE, "omk_batch_set_roots: upload the forest first");
    for (int32_t t = 0; t < n; t++)
        if (h_roots[t] < 0 || h_roots[t] >= f->n_nodes)
            return fail(OMK_ERR_INVALID, "omk_batch_set_roots: root %d of traversal %d outside [0, %lld)", h_roots[t],
                        t, (long long)f->n_nodes);
    // level-0 work items: traversals grouped by root, ascending traversal index inside a group
    std::vector<int32_t> order((size_t)n);
    for (int32_t t = 0; t < n; t++) order[(size_t)t] = t;
    std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t c) { return h_roots[a] < h_roots[c]; });
    std::vector<Item> items, singles;
    for (int32_t i = 0; i < n;) {
        int32_t j = i;
        while (j < n && h_roots[order[(size_t)j]] == h_roots[order[(size_t)i]]) j++;
        Item it;
        memset(&it, 0, sizeof(it));
        it.node = h_roots[order[(size_t)i]];
        if (j - i > 1) {
            it.off = i;
            it.m = j - i;
            items.push_back(it);
        } else {
            it.off = order[(size_t)i];  // the traversal itself
            it.m = 1;
            singles.push_back(it);
        }
        i = j;
    }
    // the most crowded roots head the longest chains of work: start them first
    std::stable_sort(items.begin(), items.end(), [](const Item &x, const Item &y) { return x.m > y.m; });
    // A root that will be cut into slices (kHeavyMin visitors or more): its boundaries depend on its statistics
    // only, so they are queued right behind the roots (items of kind 4, see prefetch_boundaries in
    // omk_select.hip) and worked out by other wavefronts while the root's own wavefront still loads its children.
    int32_t n_hctx0 = 0;
    {
        const size_t n_roots = items.size();
        for (size_t i = 0; i < n_roots && items[i].m >= kHeavyMin && n_hctx0 < b->hctx_cap; i++) {
            const int32_t S = slice_size(items[i].m), K = (items[i].m + S - 1) / S;
            if (items.size() + (size_t)K > (size_t)b->stride) break;  // (items0 holds one item per traversal)
            items[i].pad[1] = n_hctx0 + 1;
            for (int32_t bnd = 1; bnd <= K; bnd++) {
                Item it = items[i];
                it.off = 0;
                it.pad[0] = 4;
                it.pad[1] = n_hctx0;
                it.pad[2] = bnd | (S << 8);
                items.push_back(it);
            }
            n_hctx0++;
        }
    }
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipStreamSynchronize(f->stream));
    HIP_TRY(hipMemcpy(b->seg0, order.data(), (size_t)n * 4, hipMemcpyHostToDevice));
    // every path starts at its root: written here once, not by every selection (the wavefront that takes a
    // crowded root would spend its first microseconds on thousands of path entries)
    HIP_TRY(hipMemcpy(b->paths, h_roots, (size_t)n * 4, hipMemcpyHostToDevice));
    if (!items.empty())
        HIP_TRY(hipMemcpy(b->items0, items.data(), items.size() * sizeof(Item), hipMemcpyHostToDevice));
    if (!singles.empty())
        HIP_TRY(hipMemcpy(b->singles0, singles.data(), singles.size() * sizeof(Item), hipMemcpyHostToDevice));
    b->n_items0 = (int32_t)items.size();
    b->n_hctx0 = n_hctx0;
    b->n_singles0 = (int32_t)singles.size();
    b->n = n;
    b->generation = f->generation;
    b->selected = false;
    return OMK_OK;
}

int omk_batch_set_values(omk_batch *b, const float *h_values, int32_t n) {
    if (!b || !h_values) return fail(OMK_ERR_INVALID, "omk_batch_set_values: null argument");
    if (n <= 0 || n > b->max_traversals) return fail(OMK_ERR_CAPACITY, "omk_batch_set_values: %d values", n);
    if (int rc = use_device(b->f)) return rc;
    HIP_TRY(hipMemcpyAsync(b->values, h_values, (size_t)n * 4, hipMemcpyHostToDevice, b->f->stream));
    HIP_TRY(hipStreamSynchronize(b->f->stream));
    return OMK_OK;
}

int omk_batch_device(omk_batch *b, omk_batch_dev *out) {
    if (!b || !out) return fail(OMK_ERR_INVALID, "omk_batch_device: null argument");
    out->d_paths = b->paths;
    out->d_path_len = b->path_len;
    out->d_leaf = b->leaf;
    out->d_values = b->values;
    out->stride = b->stride;
    out->max_depth = b->max_depth;
    out->n_traversals = b->n;
    return OMK_OK;
}

// The number of the select call on the batch: ready marks of the queues are call numbers (the boundary table's:
// twice that), so they start over before they repeat.
static int next_epoch(omk_batch *b) {
    omk_forest *f = b->f;
    if (b->epoch >= (1 << 30) - 2) {
        HIP_TRY(launch_fill_words(b->q_ready, 0u, b->q_cap, f->stream));
        HIP_TRY(launch_fill_words(b->single_ready, 0u, b->max_traversals, f->stream));
        HIP_TRY(launch_fill_words(b->hbound, 0u, (int64_t)b->hctx_cap * kMaxSlices * kBoundInts, f->stream));
        HIP_TRY(launch_fill_words(b->hctx, 0u, (int64_t)b->hctx_cap * kHeavyCtxInts, f->stream));
        // the two depth-cap counters take turns by call parity, which this restart breaks once
        HIP_TRY(launch_fill_words(b->counters + kTruncatedWord, 0u, 2, f->stream));
        b->epoch = 0;
    }
    b->epoch++;
    return OMK_OK;
}

int omk_select_batch(omk_batch *b, const omk_select_params *p) {
    if (!b || !p) return fail(OMK_ERR_INVALID, "omk_select_batch: null argument");
    omk_forest *f = b->f;
    if (!f->uploaded || b->n <= 0) return fail(OMK_ERR_STATE, "omk_select_batch: upload a forest and set roots first");
    if (int rc = fresh_batch("omk_select_batch", b)) return rc;
    if (int rc = tree_only("omk_select_batch", f)) return rc;
    if (p->use_rave && !f->has_rave)
        return fail(OMK_ERR_INVALID, "omk_select_batch: use_rave on a forest created without RAVE arrays");
    if (p->pw && !f->prior_sorted)
        return fail(OMK_ERR_UNSUPPORTED,
                    "omk_select_batch: progressive widening needs children stored in prior-descending order "
                    "and no legal mask");
    if (int rc = use_device(f)) return rc;
    if (p->use_rave && (!f->blend_valid || !f->blend_k_known || f->blend_k != p->rave_k)) {
        HIP_TRY(launch_blend_all(f->dev(), p->rave_k, f->stream));
        f->blend_valid = f->blend_k_known = true;
        f->blend_k = p->rave_k;
    }
    SelectArgs a;
    memset(&a, 0, sizeof(a));
    a.items0 = b->items0;
    a.seg0 = b->seg0;
    a.items_q = b->items_q;
    a.seg[0] = b->seg[0];
    a.seg[1] = b->seg[1];
    if (int rc = next_epoch(b)) return rc;
    a.q_ready = b->q_ready;
    a.q_cap = b->q_cap;
    a.epoch = b->epoch;
    a.spin_limit = b->spin_limit;
    a.truncated = b->counters + kTruncatedWord + (b->epoch & 1);
    a.truncated_next = b->counters + kTruncatedWord + ((b->epoch + 1) & 1);
    a.stats = b->stats_on ? b->counters + 1 : nullptr;
    a.n_singles = b->counters + 17;
    a.sched_head = b->counters + 1 * kSchedStep;
    a.sched_tail = b->counters + 2 * kSchedStep;
    a.sched_wait = b->counters + 3 * kSchedStep;
    a.singles_head = b->counters + 4 * kSchedStep;
    a.single_ready = b->single_ready;
    a.n_trav = b->n;
    a.n_team_blocks = 0;
    a.fast_singles = 0;
    // A waiting wavefront sleeps about a microsecond between two polls, so that hundreds of them leave the memory
    // system to those that work.  A small batch has few wavefronts waiting and a short chain of crowded nodes, every
    // hand-over of which pays that sleep: they poll without it (measured on 64 traversals: 0.095 -> 0.092 ms; on
    // 4096, with the sleep off: 0.216 -> 0.221).
    a.poll_sleep = b->n <= 256 ? 0 : b->poll_sleep;
    a.hctx = b->hctx;
    a.hbound = b->hbound;
    a.hctx_n = b->counters + 2 * kSchedStep + 64;
    a.hctx_cap = b->hctx_cap;
    a.list_flag = b->list_flag;
    static_assert(kHeavyCtxInts >= 16 + OMK_MAX_FANOUT, "context too small");
    a.times = b->counters + 26;
    a.trace = b->trace_on ? (long long *)b->out_paths : nullptr;  // staging that only omk_batch_read uses
    a.trace_n = b->counters + 24;
    a.trace_cap = (int32_t)(b->out_ints / 24);
    a.singles0 = b->singles0;
    a.singles_q = b->singles_q;
    a.sc_child = b->sc_child;
    a.sc_occ = b->sc_occ;
    a.paths = b->paths;
    a.path_len = b->path_len;
    a.leaf = b->leaf;
    a.stride = b->stride;
    a.max_depth = b->max_depth;
    a.vl = p->virtual_loss;
    a.pw = p->pw;
    a.c_puct = p->c_puct;
    a.rave_k = p->rave_k;
    HIP_TRY(launch_select(f->dev(), a, b->n_items0, b->n_singles0, b->n, f->max_fanout, p->use_rave != 0, b->n_cus,
                          b->n_hctx0, f->stream));
    b->selected = true;
    return OMK_OK;
}

int omk_backup_batch(omk_batch *b, int32_t virtual_loss) {
    if (!b) return fail(OMK_ERR_INVALID, "omk_backup_batch: null batch");
    if (!b->selected) return fail(OMK_ERR_STATE, "omk_backup_batch: no selected paths");
    if (int rc = fresh_batch("omk_backup_batch", b)) return rc;
    if (int rc = use_device(b->f)) return rc;
    HIP_TRY(launch_backup(b->f->dev(), b->paths, b->path_len, b->values, b->n, b->stride, b->max_depth + 1,
                          virtual_loss, b->f->stream));
    // N and W of the nodes on the paths have changed: their RAVE blend with them
    if (b->f->has_rave && b->f->blend_valid)
        HIP_TRY(launch_blend_paths(b->f->dev(), b->paths, b->path_len, b->n, b->stride, b->max_depth + 1, b->f->blend_k,
                                   b->f->stream));
    return OMK_OK;
}

int omk_backup_rave_batch(omk_batch *b) {
    if (!b) return fail(OMK_ERR_INVALID, "omk_backup_rave_batch: null batch");
    if (!b->selected) return fail(OMK_ERR_STATE, "omk_backup_rave_batch: no selected paths");
    if (int rc = fresh_batch("omk_backup_rave_batch", b)) return rc;
    if (!b->f->has_rave) return fail(OMK_ERR_INVALID, "omk_backup_rave_batch: the forest has no RAVE arrays");
    if (int rc = tree_only("omk_backup_rave_batch", b->f)) return rc;
    if (int rc = use_device(b->f)) return rc;
    HIP_TRY(launch_rave_backup(b->f->mut(), b->paths, b->path_len, b->values, b->n, b->stride, b->max_depth + 1,
                               b->f->stream));
    b->f->blend_valid = false;  // rN and rW of children of path nodes have changed: the next selection starts over
    return OMK_OK;
}

int omk_revert_vl(omk_batch *b, int32_t virtual_loss) {
    if (!b) return fail(OMK_ERR_INVALID, "omk_revert_vl: null batch");
    if (!b->selected) return fail(OMK_ERR_STATE, "omk_revert_vl: no selected paths");
    if (int rc = fresh_batch("omk_revert_vl", b)) return rc;
    if (int rc = use_device(b->f)) return rc;
    HIP_TRY(launch_revert_vl(b->f->dev(), b->paths, b->path_len, b->n, b->stride, b->max_depth + 1, virtual_loss,
                             b->f->stream));
    return OMK_OK;
}

static int check_paths_args(const char *who, omk_forest *f, const void *paths, const void *len, int32_t n,
                            int32_t stride, int32_t max_len) {
    if (!f || !paths || !len) return fail(OMK_ERR_INVALID, "%s: null argument", who);
    if (!f->uploaded) return fail(OMK_ERR_STATE, "%s: upload the forest first", who);
    if (n < 0 || stride < n || max_len < 0 || max_len > 4097)
        return fail(OMK_ERR_INVALID, "%s: n %d stride %d max_len %d", who, n, stride, max_len);
    return use_device(f);
}

int omk_apply_vl_paths(omk_forest *f, const int32_t *d_paths, const int32_t *d_path_len, int32_t n, int32_t stride,
                       int32_t max_len, int32_t virtual_loss) {
    if (int rc = check_paths_args("omk_apply_vl_paths", f, d_paths, d_path_len, n, stride, max_len)) return rc;
    HIP_TRY(launch_apply_vl(f->dev(), d_paths, d_path_len, n, stride, max_len, virtual_loss, f->stream));
    return OMK_OK;
}

int omk_revert_vl_paths(omk_forest *f, const int32_t *d_paths, const int32_t *d_path_len, int32_t n, int32_t stride,
                        int32_t max_len, int32_t virtual_loss) {
    if (int rc = check_paths_args("omk_revert_vl_paths", f, d_paths, d_path_len, n, stride, max_len)) return rc;
    HIP_TRY(launch_revert_vl(f->dev(), d_paths, d_path_len, n, stride, max_len, virtual_loss, f->stream));
    return OMK_OK;
}

int omk_backup_paths(omk_forest *f, const int32_t *d_paths, const int32_t *d_path_len, const float *d_values,
                     int32_t n, int32_t stride, int32_t max_len, int32_t virtual_loss) {
    if (int rc = check_paths_args("omk_backup_paths", f, d_paths, d_path_len, n, stride, max_len)) return rc;
    if (!d_values) return fail(OMK_ERR_INVALID, "omk_backup_paths: null values");
    HIP_TRY(launch_backup(f->dev(), d_paths, d_path_len, d_values, n, stride, max_len, virtual_loss, f->stream));
    if (f->has_rave && f->blend_valid)
        HIP_TRY(launch_blend_paths(f->dev(), d_paths, d_path_len, n, stride, max_len, f->blend_k, f->stream));
    return OMK_OK;
}

// How many children MCTSNode::expand creates for a node of `visits` visits that is offered `legal`
// moves (src/mcts/mcts_node.cpp:296-341): without progressive widening all of them; with it
// min(legal, size_t(max(8.0f, float(cpw * std::pow(visits + 1, kpw))))), at least 1.  (std::pow of an
// int and a float is computed in double; the product with the float cpw as well.)  The branch of
// expand() that adds children to a node that already has some is never reached: the
// compare-exchange on is_expanded_ at :264 returns first.
static int32_t widened_children(int32_t legal, int32_t visits, const omk_expand_params *p) {
    if (!p || !p->use_progressive_widening) return legal;
    const double grown = (double)p->progressive_widening_c * std::pow((double)(visits + 1), (double)p->progressive_widening_k);
    const float target_f = std::max(8.0f, static_cast<float>(grown));
    // a float beyond the range of size_t is undefined in the reference; every such value exceeds `legal`
    size_t target = target_f >= 1.0e18f ? (size_t)legal : static_cast<size_t>(target_f);
    if (!(target_f == target_f)) target = 8;  // NaN: std::max(8.0f, NaN) is 8.0f
    size_t num = std::min((size_t)legal, target);
    num = std::max(num, (size_t)1);
    return (int32_t)std::min(num, (size_t)legal);
}

int omk_expand_batch_ex(omk_batch *b, const int32_t *h_move_begin, const int32_t *h_moves, const int32_t *h_policy_begin,
                        const float *h_policy, const omk_expand_params *params, int32_t *h_first_child) {
    if (!b || !h_move_begin || !h_moves || !params) return fail(OMK_ERR_INVALID, "omk_expand_batch_ex: null argument");
    if (!b->selected) return fail(OMK_ERR_STATE, "omk_expand_batch_ex: no selected paths");
    if (int rc = fresh_batch("omk_expand_batch_ex", b)) return rc;
    if ((h_policy != nullptr) != (h_policy_begin != nullptr))
        return fail(OMK_ERR_INVALID, "omk_expand_batch_ex: policies need both their values and their offsets");
    const int32_t action_space = params->action_space;
    if (h_policy && action_space <= 0)
        return fail(OMK_ERR_INVALID, "omk_expand_batch_ex: a policy needs action_space > 0 (got %d)", action_space);
    omk_forest *f = b->f;
    if (int rc = use_device(f)) return rc;
    hipStream_t s = f->stream;
    const int n = b->n;
    std::vector<int32_t> leaf((size_t)n);
    HIP_TRY(hipMemcpyAsync(leaf.data(), b->leaf, (size_t)n * 4, hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    // one job per distinct leaf: the first traversal (in index order) that offers moves wins
    std::vector<ExpandJob> jobs;
    std::vector<int32_t> job_of((size_t)n, -1), moves;
    std::vector<float> priors;
    {
        std::vector<std::pair<int32_t, int32_t>> order;  // (leaf, traversal) of every offer
        for (int t = 0; t < n; t++) {
            if (h_move_begin[t + 1] < h_move_begin[t])
                return fail(OMK_ERR_INVALID, "omk_expand_batch_ex: move_begin decreases at traversal %d", t);
            if (h_policy_begin && h_policy_begin[t + 1] < h_policy_begin[t])
                return fail(OMK_ERR_INVALID, "omk_expand_batch_ex: policy_begin decreases at traversal %d", t);
            if (h_move_begin[t + 1] > h_move_begin[t] && leaf[(size_t)t] >= 0) order.emplace_back(leaf[(size_t)t], t);
        }
        std::sort(order.begin(), order.end());
        std::vector<int32_t> winners;
        for (size_t i = 0; i < order.size(); i++)
            if (i == 0 || order[i].first != order[i - 1].first) winners.push_back(order[i].second);
        std::sort(winners.begin(), winners.end());  // ids are handed out in traversal order
        // A leaf that has children already (the selection stopped at it because of the depth bound) is left alone
        // and takes no ids: its child range is read first.  Progressive widening reads the visit count of every
        // leaf that is about to be expanded: it comes in the same trip.
        std::vector<int32_t> visits(winners.size(), 0);
        if (!winners.empty()) {
            const size_t nw = winners.size();
            if (nw * 16 > b->exp_bytes) {
                if (b->exp_buf) HIP_TRY(hipFree(b->exp_buf));
                b->exp_buf = nullptr;
                b->exp_bytes = 0;
                HIP_TRY(hipMalloc(&b->exp_buf, nw * 32));
                b->exp_bytes = nw * 32;
            }
            std::vector<int32_t> ids(nw);
            std::vector<int2> spans(nw);
            for (size_t i = 0; i < nw; i++) ids[i] = leaf[(size_t)winners[i]];
            int32_t *d_ids = (int32_t *)b->exp_buf, *d_n = d_ids + nw;
            uint64_t *d_span = (uint64_t *)(d_ids + 2 * nw);
            HIP_TRY(hipMemcpyAsync(d_ids, ids.data(), nw * 4, hipMemcpyHostToDevice, s));
            HIP_TRY(launch_gather_words((uint32_t *)d_n, (const uint32_t *)f->N, d_ids, (int64_t)nw, s));
            HIP_TRY(launch_gather_dwords(d_span, (const uint64_t *)f->span, d_ids, (int64_t)nw, s));
            HIP_TRY(hipMemcpyAsync(visits.data(), d_n, nw * 4, hipMemcpyDeviceToHost, s));
            HIP_TRY(hipMemcpyAsync(spans.data(), d_span, nw * 8, hipMemcpyDeviceToHost, s));
            HIP_TRY(hipStreamSynchronize(s));
            size_t kept = 0;
            for (size_t i = 0; i < nw; i++) {
                if (spans[i].y != 0) continue;
                winners[kept] = winners[i];
                visits[kept] = visits[i];
                kept++;
            }
            winners.resize(kept);
            visits.resize(kept);
        }
        int64_t cursor = f->n_nodes;
        bool sorted = true;
        int mf = f->max_fanout;
        for (size_t wi = 0; wi < winners.size(); wi++) {
            const int32_t t = winners[wi];
            int32_t cnt = h_move_begin[t + 1] - h_move_begin[t];
            if (cnt > 1000) cnt = 1000;  // MCTSNode::expand: max_reasonable_moves
            cnt = widened_children(cnt, visits[wi], params);
            // MCTSNode::setPriorProbabilities (:512-593) is only called with a policy that is not empty
            // (mcts_engine_batch_tree_simple.cpp:256-258); otherwise expand's uniform prior stays
            const int32_t psize = h_policy_begin ? h_policy_begin[t + 1] - h_policy_begin[t] : 0;
            const float *pol = psize > 0 ? h_policy + h_policy_begin[t] : nullptr;
            ExpandJob j;
            j.leaf = leaf[(size_t)t];
            j.begin = (int32_t)cursor;
            j.count = cnt;
            j.off = (int32_t)moves.size();
            float prev = 2.0f;
            for (int32_t i = 0; i < cnt; i++) {
                const int32_t mv = h_moves[h_move_begin[t] + i];
                float prior;
                if (!pol) {
                    prior = 1.0f / (float)cnt;  // expand(): uniform prior
                } else if (psize == action_space) {  // a policy over the action space (:537-560)
                    if (mv >= 0 && mv < action_space) {
                        prior = pol[mv];
                        prior = std::min(1.0f, std::max(0.0f, prior));  // clamp to [0, 1]
                    } else {
                        prior = 0.01f;  // move outside the action space
                    }
                } else if (psize == cnt) {  // one value per child, by child index (:561-575)
                    prior = pol[i];
                    prior = std::min(1.0f, std::max(0.0f, prior));
                } else {  // neither size: uniform (:576-584)
                    prior = 1.0f / (float)cnt;
                }
                if (prior > prev) sorted = false;
                prev = prior;
                moves.push_back(mv);
                priors.push_back(prior);
            }
            job_of[(size_t)t] = (int32_t)jobs.size();
            jobs.push_back(j);
            cursor += cnt;
            mf = std::max(mf, (int)cnt);
        }
        if (cursor > f->capacity)
            return fail(OMK_ERR_CAPACITY, "omk_expand_batch_ex: %lld nodes needed, capacity %lld", (long long)cursor,
                        (long long)f->capacity);
        if (cursor > INT32_MAX) return fail(OMK_ERR_CAPACITY, "omk_expand_batch_ex: node ids exceed 32 bits");
        if (h_first_child)
            for (int t = 0; t < n; t++) h_first_child[t] = -1;
        if (jobs.empty()) return OMK_OK;
        // staging: jobs | moves | priors | status
        const size_t nj = jobs.size(), nm = moves.size();
        const size_t bytes = nj * sizeof(ExpandJob) + nm * 8 + nj * 4;
        if (bytes > b->exp_bytes) {
            if (b->exp_buf) HIP_TRY(hipFree(b->exp_buf));
            b->exp_buf = nullptr;
            b->exp_bytes = 0;
            HIP_TRY(hipMalloc(&b->exp_buf, bytes * 2));
            b->exp_bytes = bytes * 2;
        }
        char *base = (char *)b->exp_buf;
        ExpandJob *d_jobs = (ExpandJob *)base;
        int32_t *d_moves = (int32_t *)(base + nj * sizeof(ExpandJob));
        float *d_priors = (float *)(d_moves + nm);
        int32_t *d_status = (int32_t *)(d_priors + nm);
        HIP_TRY(hipMemcpyAsync(d_jobs, jobs.data(), nj * sizeof(ExpandJob), hipMemcpyHostToDevice, s));
        HIP_TRY(hipMemcpyAsync(d_moves, moves.data(), nm * 4, hipMemcpyHostToDevice, s));
        HIP_TRY(hipMemcpyAsync(d_priors, priors.data(), nm * 4, hipMemcpyHostToDevice, s));
        HIP_TRY(launch_expand(f->mut(), d_jobs, (int)nj, d_moves, d_priors, d_status, f->n_nodes, cursor, s));
        std::vector<int32_t> status(nj);
        HIP_TRY(hipMemcpyAsync(status.data(), d_status, nj * 4, hipMemcpyDeviceToHost, s));
        HIP_TRY(hipStreamSynchronize(s));
        f->n_nodes = cursor;
        f->structure_changed = true;  // ids keep their meaning, but an upload of the old arrays would not
        f->max_fanout = mf;
        if (!sorted) f->prior_sorted = false;
        if (h_first_child)
            for (int t = 0; t < n; t++)
                if (job_of[(size_t)t] >= 0) h_first_child[t] = status[(size_t)job_of[(size_t)t]];
    }
    return OMK_OK;
}

int omk_expand_batch(omk_batch *b, const int32_t *h_move_begin, const int32_t *h_moves, const float *h_policy,
                     int32_t action_space, int32_t *h_first_child) {
    if (!b || !h_move_begin || !h_moves) return fail(OMK_ERR_INVALID, "omk_expand_batch: null argument");
    if (h_policy && action_space <= 0)
        return fail(OMK_ERR_INVALID, "omk_expand_batch: a policy needs action_space > 0 (got %d)", action_space);
    omk_expand_params p;
    p.action_space = action_space;
    p.use_progressive_widening = 0;
    p.progressive_widening_c = 0.0f;
    p.progressive_widening_k = 0.0f;
    std::vector<int32_t> pb;
    if (h_policy) {  // one row of action_space values per traversal
        pb.resize((size_t)b->n + 1);
        for (int32_t t = 0; t <= b->n; t++) pb[(size_t)t] = t * action_space;
    }
    return omk_expand_batch_ex(b, h_move_begin, h_moves, h_policy ? pb.data() : nullptr, h_policy, &p, h_first_child);
}

int omk_batch_read(omk_batch *b, int32_t *h_paths, int32_t *h_path_len, int32_t *h_leaf, int32_t *h_actions) {
    if (!b) return fail(OMK_ERR_INVALID, "omk_batch_read: null batch");
    if (!b->selected) return fail(OMK_ERR_STATE, "omk_batch_read: no selected paths");
    if (int rc = fresh_batch("omk_batch_read", b)) return rc;
    omk_forest *f = b->f;
    if (int rc = use_device(f)) return rc;
    hipStream_t s = f->stream;
    const int n = b->n, D = b->max_depth;
    if (h_paths || h_actions)
        HIP_TRY(launch_export(f->dev(), b->paths, b->path_len, n, b->stride, D, h_paths ? b->out_paths : nullptr,
                              h_actions ? b->out_actions : nullptr, s));
    if (h_paths) HIP_TRY(hipMemcpyAsync(h_paths, b->out_paths, (size_t)n * (D + 1) * 4, hipMemcpyDeviceToHost, s));
    if (h_actions) HIP_TRY(hipMemcpyAsync(h_actions, b->out_actions, (size_t)n * D * 4, hipMemcpyDeviceToHost, s));
    if (h_path_len) HIP_TRY(hipMemcpyAsync(h_path_len, b->path_len, (size_t)n * 4, hipMemcpyDeviceToHost, s));
    if (h_leaf) HIP_TRY(hipMemcpyAsync(h_leaf, b->leaf, (size_t)n * 4, hipMemcpyDeviceToHost, s));
    int32_t ab[4] = {0, 0, 0, 0};  // abort flag and what the wavefront that raised it was waiting for
    HIP_TRY(hipMemcpyAsync(ab, b->counters + 3 * kSchedStep + 1, sizeof(ab), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    if (ab[0] == 1)
        return fail(OMK_ERR_STATE,
                    "omk_batch_read: the selection gave up (a wavefront waited longer than the spin limit for item %d "
                    "of the work queue, %d handed out, %d visitors open); its paths are incomplete, revert the virtual "
                    "losses with omk_forest_upload or omk_revert_vl_paths over known paths",
                    ab[1], ab[2], ab[3]);
    if (ab[0] == 3)
        return fail(OMK_ERR_STATE,
                    "omk_batch_read: the selection gave up (a wavefront waited longer than the spin limit for the "
                    "visitor list at %d of depth %d, complete to depth %d); its paths are incomplete, revert the "
                    "virtual losses with omk_forest_upload or omk_revert_vl_paths over known paths",
                    ab[1], ab[2], ab[3]);
    if (ab[0] == 4)
        return fail(OMK_ERR_STATE,
                    "omk_batch_read: the selection gave up (a wavefront waited longer than the spin limit for entry %d "
                    "of the single-visitor queue, %d written, %d visitors open); its paths are incomplete, revert the "
                    "virtual losses with omk_forest_upload or omk_revert_vl_paths over known paths",
                    ab[1], ab[2], ab[3]);
    if (ab[0])
        return fail(OMK_ERR_STATE,
                    "omk_batch_read: the selection gave up (work queue overflow); its paths are incomplete, revert "
                    "the virtual losses with omk_forest_upload or omk_revert_vl_paths over known paths");
    return OMK_OK;
}

int omk_batch_truncated(omk_batch *b, int32_t *h_count) {
    if (!b || !h_count) return fail(OMK_ERR_INVALID, "omk_batch_truncated: null argument");
    if (!b->selected) return fail(OMK_ERR_STATE, "omk_batch_truncated: no selected paths");
    if (int rc = use_device(b->f)) return rc;
    HIP_TRY(hipMemcpyAsync(h_count, b->counters + kTruncatedWord + (b->epoch & 1), 4, hipMemcpyDeviceToHost,
                           b->f->stream));
    HIP_TRY(hipStreamSynchronize(b->f->stream));
    return OMK_OK;
}

int omk_batch_set_stats(omk_batch *b, int32_t enabled) {
    if (!b) return fail(OMK_ERR_INVALID, "omk_batch_set_stats: null batch");
    b->stats_on = enabled != 0;
    return OMK_OK;
}

int omk_batch_set_spin_limit(omk_batch *b, int32_t polls) {
    if (!b) return fail(OMK_ERR_INVALID, "omk_batch_set_spin_limit: null batch");
    if (polls < 0) return fail(OMK_ERR_INVALID, "omk_batch_set_spin_limit: polls %d", polls);
    b->spin_limit = polls;
    return OMK_OK;
}

int omk_debug_set_select_count(omk_batch *b, int32_t count) {
    if (!b) return fail(OMK_ERR_INVALID, "omk_debug_set_select_count: null batch");
    if (count < b->epoch || count >= (1 << 30))
        return fail(OMK_ERR_INVALID, "omk_debug_set_select_count: count %d (the last call was number %d; forward only, "
                    "below 2^30)", count, b->epoch);
    // the two depth-cap counters take turns by call parity: keep the parity, so that the counter the next call
    // starts from is the one the last call cleared
    if ((count & 1) != (b->epoch & 1)) {
        if (count + 1 >= (1 << 30)) return fail(OMK_ERR_INVALID, "omk_debug_set_select_count: count %d", count);
        count++;
    }
    b->epoch = count;
    return OMK_OK;
}

int omk_batch_stats(omk_batch *b, int32_t *h_stats16) {
    int32_t *h_stats8 = h_stats16;
    if (!b || !h_stats8) return fail(OMK_ERR_INVALID, "omk_batch_stats: null argument");
    if (!b->selected) return fail(OMK_ERR_STATE, "omk_batch_stats: no selected paths");
    if (int rc = use_device(b->f)) return rc;
    HIP_TRY(hipMemcpyAsync(h_stats8, b->counters + 1, 64, hipMemcpyDeviceToHost, b->f->stream));
    int32_t times[3] = {0, 0, 0};
    HIP_TRY(hipMemcpyAsync(times, b->counters + 26, sizeof(times), hipMemcpyDeviceToHost, b->f->stream));
    HIP_TRY(hipStreamSynchronize(b->f->stream));
    // the three time stamps are kept whether or not the counters are on
    for (int i = 0; i < 3; i++) h_stats8[8 + i] = times[i];
    return OMK_OK;
}

// The per-node timeline of the last selection (12 x int64 per processed multi-visitor item), recorded when
// omk_batch_set_trace switched it on before that selection.
int omk_debug_trace(omk_batch *b, long long *h_trace, int32_t max_entries, int32_t *h_n) {
    if (!b || !h_trace || !h_n || max_entries < 0) return fail(OMK_ERR_INVALID, "omk_debug_trace: bad argument");
    *h_n = 0;
    if (!b->trace_on) return fail(OMK_ERR_STATE, "omk_debug_trace: switch the timeline on first (omk_batch_set_trace)");
    if (!b->selected) return fail(OMK_ERR_STATE, "omk_debug_trace: no selected paths");
    if (int rc = use_device(b->f)) return rc;
    HIP_TRY(hipStreamSynchronize(b->f->stream));
    HIP_TRY(hipMemcpy(h_n, b->counters + 24, 4, hipMemcpyDeviceToHost));
    int32_t n = std::min(std::min(*h_n, max_entries), (int32_t)(b->out_ints / 24));
    if (n > 0) HIP_TRY(hipMemcpy(h_trace, b->out_paths, (size_t)n * 96, hipMemcpyDeviceToHost));
    *h_n = n;
    return OMK_OK;
}

int omk_batch_set_trace(omk_batch *b, int32_t enabled) {
    if (!b) return fail(OMK_ERR_INVALID, "omk_batch_set_trace: null batch");
    b->trace_on = enabled != 0;
    return OMK_OK;
}

// ---------------------------------------------------------------- transposition table

int omk_tt_create(omk_forest *f, int32_t log2_slots, omk_tt **out) {
    if (!f || !out) return fail(OMK_ERR_INVALID, "omk_tt_create: null argument");
    if (log2_slots < 4 || log2_slots > 30) return fail(OMK_ERR_INVALID, "omk_tt_create: log2_slots %d", log2_slots);
    if (int rc = use_device(f)) return rc;
    omk_tt *tt = new (std::nothrow) omk_tt();
    if (!tt) return fail(OMK_ERR_INVALID, "out of host memory");
    tt->f = f;
    f->children++;
    tt->log2_slots = log2_slots;
    hipError_t e = dalloc(&tt->slots, 1ll << log2_slots);
    if (e == hipSuccess) e = dalloc(&tt->meta, 1ll << log2_slots);
    if (e == hipSuccess) e = dalloc(&tt->d_status, 8);
    if (e != hipSuccess) {
        int rc = fail(OMK_ERR_HIP, "omk_tt_create: %s", hipGetErrorString(e));
        omk_tt_destroy(tt);
        return rc;
    }
    *out = tt;
    return omk_tt_clear(tt);
}

int omk_tt_destroy(omk_tt *tt) {
    if (!tt) return OMK_OK;
    (void)hipSetDevice(tt->f->device);
    (void)hipStreamSynchronize(tt->f->stream);
    if (tt->slots) (void)hipFree(tt->slots);
    if (tt->meta) (void)hipFree(tt->meta);
    if (tt->work) (void)hipFree(tt->work);
    if (tt->d_status) (void)hipFree(tt->d_status);
    (void)hipGetLastError();
    forest_child_gone(tt->f);
    delete tt;
    return OMK_OK;
}

int omk_tt_clear(omk_tt *tt) {
    if (!tt) return fail(OMK_ERR_INVALID, "omk_tt_clear: null table");
    if (int rc = use_device(tt->f)) return rc;
    HIP_TRY(launch_tt_clear(tt->slots, tt->meta, tt->log2_slots, tt->f->stream));
    tt->clock = 0;
    tt->generation = -1;
    return OMK_OK;
}

int omk_tt_insert(omk_tt *tt, const uint64_t *d_keys, const int32_t *d_nodes, const int32_t *d_depths, int64_t n) {
    if (!tt || !d_keys || !d_nodes) return fail(OMK_ERR_INVALID, "omk_tt_insert: null argument");
    if (n < 0) return fail(OMK_ERR_INVALID, "omk_tt_insert: n %lld", (long long)n);
    if (int rc = use_device(tt->f)) return rc;
    if (int rc = tt_same_tree(tt)) return rc;
    hipStream_t s = tt->f->stream;
    int status[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    HIP_TRY(hipMemcpyAsync(tt->d_status, status, sizeof(status), hipMemcpyHostToDevice, s));
    HIP_TRY(launch_tt_insert(tt->slots, tt->log2_slots, d_keys, d_nodes, d_depths, n, tt->d_status, s));
    HIP_TRY(hipMemcpyAsync(status, tt->d_status, sizeof(status), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    if (status[1]) return fail(OMK_ERR_INVALID, "omk_tt_insert: %d keys equal the empty marker ~0", status[1]);
    if (status[0]) return fail(OMK_ERR_CAPACITY, "omk_tt_insert: table full, %d entries dropped", status[0]);
    return OMK_OK;
}

int omk_tt_probe(omk_tt *tt, const uint64_t *d_keys, int64_t n, int32_t min_depth, int32_t *d_out) {
    if (!tt || !d_keys || !d_out) return fail(OMK_ERR_INVALID, "omk_tt_probe: null argument");
    if (n < 0) return fail(OMK_ERR_INVALID, "omk_tt_probe: n %lld", (long long)n);
    if (int rc = use_device(tt->f)) return rc;
    if (int rc = tt_same_tree(tt)) return rc;
    HIP_TRY(launch_tt_probe(tt->slots, tt->log2_slots, d_keys, nullptr, nullptr, 0, n, min_depth, d_out, tt->meta,
                            tt->clock, tt->f->stream));
    tt->clock += (uint32_t)n;
    return OMK_OK;
}

int omk_tt_probe_leaves(omk_tt *tt, omk_batch *b, int32_t min_depth, int32_t *d_out) {
    if (!tt || !b || !d_out) return fail(OMK_ERR_INVALID, "omk_tt_probe_leaves: null argument");
    if (tt->f != b->f) return fail(OMK_ERR_INVALID, "omk_tt_probe_leaves: table and batch belong to different forests");
    if (!b->selected) return fail(OMK_ERR_STATE, "omk_tt_probe_leaves: no selected paths");
    if (int rc = fresh_batch("omk_tt_probe_leaves", b)) return rc;
    if (!b->f->has_hash) return fail(OMK_ERR_STATE, "omk_tt_probe_leaves: the forest was uploaded without position keys");
    if (int rc = use_device(tt->f)) return rc;
    if (int rc = tt_same_tree(tt)) return rc;
    HIP_TRY(launch_tt_probe(tt->slots, tt->log2_slots, nullptr, b->leaf, b->f->hash, b->f->n_nodes, b->n, min_depth, d_out,
                            tt->meta, tt->clock, tt->f->stream));
    tt->clock += (uint32_t)b->n;
    return OMK_OK;
}

int omk_tt_set_replacement_threshold(omk_tt *tt, float threshold) {
    if (!tt || !(threshold >= 0.0f)) return fail(OMK_ERR_INVALID, "omk_tt_set_replacement_threshold: bad argument");
    tt->threshold = threshold;
    return OMK_OK;
}

static int tt_report(const char *who, const int *st, int32_t *h_counts) {
    if (h_counts) {
        h_counts[0] = st[3];  // new entries
        h_counts[1] = st[4];  // replacements
        h_counts[2] = st[2];  // later entries of the call with a key an earlier one carries: dropped
        h_counts[3] = st[6];  // transpositions reported (traverse)
    }
    if (st[1]) return fail(OMK_ERR_INVALID, "%s: %d keys equal the empty marker ~0", who, st[1]);
    if (st[0]) return fail(OMK_ERR_CAPACITY, "%s: table full, %d entries dropped", who, st[0]);
    return OMK_OK;
}

int omk_tt_store(omk_tt *tt, const uint64_t *d_keys, const int32_t *d_nodes, const int32_t *d_depths, int64_t n,
                 int32_t *h_counts) {
    if (!tt || !d_keys || !d_nodes) return fail(OMK_ERR_INVALID, "omk_tt_store: null argument");
    if (n < 0 || n > (1ll << 30)) return fail(OMK_ERR_INVALID, "omk_tt_store: n %lld", (long long)n);
    if (!tt->f->uploaded) return fail(OMK_ERR_STATE, "omk_tt_store: upload the forest first");
    if (int rc = use_device(tt->f)) return rc;
    if (int rc = tt_same_tree(tt)) return rc;
    if (int rc = tt_work(tt, (size_t)std::max<int64_t>(n, 1) * 8)) return rc;
    hipStream_t s = tt->f->stream;
    int status[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    HIP_TRY(hipMemcpyAsync(tt->d_status, status, sizeof(status), hipMemcpyHostToDevice, s));
    HIP_TRY(launch_tt_store(tt->f->dev(), tt->slots, tt->meta, tt->log2_slots, d_keys, d_nodes, d_depths, n,
                            (int64_t *)tt->work, tt->clock, tt->threshold, tt->d_status, s));
    tt->clock += (uint32_t)n;
    HIP_TRY(hipMemcpyAsync(status, tt->d_status, sizeof(status), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    return tt_report("omk_tt_store", status, h_counts);
}

int omk_tt_traverse(omk_tt *tt, omk_batch *b, const uint64_t *d_piece_keys, int32_t cells, const uint64_t *d_player_keys,
                    const uint64_t *d_root_keys, const int32_t *d_root_players, int32_t *d_hits, int32_t *h_counts) {
    if (!tt || !b) return fail(OMK_ERR_INVALID, "omk_tt_traverse: null argument");
    if (tt->f != b->f) return fail(OMK_ERR_INVALID, "omk_tt_traverse: table and batch belong to different forests");
    if (!b->selected) return fail(OMK_ERR_STATE, "omk_tt_traverse: no selected paths");
    if (int rc = fresh_batch("omk_tt_traverse", b)) return rc;
    omk_forest *f = b->f;
    if (d_piece_keys) {
        if (!d_player_keys || !d_root_keys || !d_root_players || cells <= 0)
            return fail(OMK_ERR_INVALID, "omk_tt_traverse: the game's key tables need player keys, root keys, root players "
                        "and cells > 0");
    } else if (!f->has_hash) {
        return fail(OMK_ERR_STATE, "omk_tt_traverse: no key tables given and the forest was uploaded without position keys");
    }
    if (int rc = use_device(f)) return rc;
    if (int rc = tt_same_tree(tt)) return rc;
    hipStream_t s = f->stream;
    const int64_t n = (int64_t)b->n * b->max_depth;
    // staging: slot_of [n] i64 | keys [n] u64 | step_nodes, store_nodes, depths, found [n] i32 each
    if (int rc = tt_work(tt, (size_t)n * 32)) return rc;
    int64_t *slot_of = (int64_t *)tt->work;
    uint64_t *keys = (uint64_t *)(slot_of + n);
    int32_t *step_nodes = (int32_t *)(keys + n), *store_nodes = step_nodes + n, *depths = store_nodes + n;
    int32_t *found = depths + n;
    int status[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    HIP_TRY(hipMemcpyAsync(tt->d_status, status, sizeof(status), hipMemcpyHostToDevice, s));
    HIP_TRY(launch_step_keys(f->dev(), b->paths, b->path_len, b->n, b->stride, b->max_depth, d_piece_keys, cells,
                             d_player_keys, d_root_keys, d_root_players, keys, step_nodes, store_nodes, depths,
                             tt->d_status, s));
    // all stores first, then all lookups: a lookup that the serial loop makes before a later step's
    // store can only miss a node without visits, and such a node is no transposition (:142)
    HIP_TRY(launch_tt_store(f->dev(), tt->slots, tt->meta, tt->log2_slots, keys, store_nodes, depths, n, slot_of,
                            tt->clock, tt->threshold, tt->d_status, s));
    tt->clock += (uint32_t)n;
    HIP_TRY(launch_tt_probe(tt->slots, tt->log2_slots, keys, nullptr, nullptr, 0, n, 0, found, tt->meta, tt->clock, s));
    tt->clock += (uint32_t)n;
    HIP_TRY(launch_tt_hits(f->dev(), step_nodes, found, n, d_hits, tt->d_status, s));
    HIP_TRY(hipMemcpyAsync(status, tt->d_status, sizeof(status), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    if (status[5])
        return fail(OMK_ERR_INVALID, "omk_tt_traverse: %d paths hold a node outside the forest or a move outside [0, %d)",
                    status[5], cells);
    status[1] = 0;  // steps that do not exist carry the empty marker on purpose
    return tt_report("omk_tt_traverse", status, h_counts);
}

int omk_tt_select_redirect(omk_tt *tt, omk_batch *b, const omk_select_params *p, int32_t *d_moves, int32_t *h_counts) {
    if (!tt || !b || !p) return fail(OMK_ERR_INVALID, "omk_tt_select_redirect: null argument");
    if (tt->f != b->f) return fail(OMK_ERR_INVALID, "omk_tt_select_redirect: table and batch belong to different forests");
    omk_forest *f = b->f;
    if (!f->uploaded || b->n <= 0)
        return fail(OMK_ERR_STATE, "omk_tt_select_redirect: upload a forest and set roots first");
    if (int rc = fresh_batch("omk_tt_select_redirect", b)) return rc;
    if (!f->has_hash)
        return fail(OMK_ERR_STATE, "omk_tt_select_redirect: the forest has no position keys (upload them, or "
                    "omk_forest_set_keys)");
    if (p->use_rave && !f->has_rave)
        return fail(OMK_ERR_INVALID, "omk_tt_select_redirect: use_rave on a forest created without RAVE arrays");
    if (p->pw)
        return fail(OMK_ERR_UNSUPPORTED, "omk_tt_select_redirect: progressive widening at selection time is not "
                    "part of this loop");
    if (int rc = use_device(f)) return rc;
    if (int rc = tt_same_tree(tt)) return rc;
    hipStream_t s = f->stream;
    if (!f->alias) {
        HIP_TRY(dalloc(&f->alias, f->capacity));
        HIP_TRY(launch_fill_words(f->alias, 0xFFFFFFFFu, f->capacity, s));
    }
    if (int rc = next_epoch(b)) return rc;
    int status[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    HIP_TRY(hipMemcpyAsync(tt->d_status, status, sizeof(status), hipMemcpyHostToDevice, s));
    RedirectArgs a;
    memset(&a, 0, sizeof(a));
    a.alias = f->alias;
    a.slots = tt->slots;
    a.meta = tt->meta;
    a.log2_slots = tt->log2_slots;
    a.t0 = tt->clock;
    a.threshold = tt->threshold;
    a.paths = b->paths;
    a.path_len = b->path_len;
    a.leaf = b->leaf;
    a.moves = d_moves;
    a.n = b->n;
    a.stride = b->stride;
    a.max_depth = b->max_depth;
    a.vl = p->virtual_loss;
    a.c_puct = p->c_puct;
    a.rave_k = p->rave_k;
    a.counts = tt->d_status;
    a.truncated = b->counters + kTruncatedWord + (b->epoch & 1);
    a.truncated_next = b->counters + kTruncatedWord + ((b->epoch + 1) & 1);
    a.abort_word = b->counters + 3 * kSchedStep + 1;
    HIP_TRY(launch_select_redirect(f->dev(), a, p->use_rave != 0, s));
    b->selected = true;
    HIP_TRY(hipMemcpyAsync(status, tt->d_status, sizeof(status), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    tt->clock += (uint32_t)status[6];  // the ticks of the access counter
    if (status[3] > 0) f->redirected = true;
    if (h_counts)
        for (int i = 0; i < 5; i++) h_counts[i] = status[i];
    if (status[5])
        return fail(OMK_ERR_CAPACITY, "omk_tt_select_redirect: table full, %d entries dropped", status[5]);
    return OMK_OK;
}

int omk_forest_download_redirects(omk_forest *f, int64_t n_nodes, int32_t *h_alias) {
    if (!f || !h_alias) return fail(OMK_ERR_INVALID, "omk_forest_download_redirects: null argument");
    if (!f->uploaded) return fail(OMK_ERR_STATE, "omk_forest_download_redirects: nothing uploaded");
    if (n_nodes != f->n_nodes)
        return fail(OMK_ERR_INVALID, "omk_forest_download_redirects: room for %lld nodes, the forest holds %lld",
                    (long long)n_nodes, (long long)f->n_nodes);
    if (!f->alias) {
        for (int64_t i = 0; i < n_nodes; i++) h_alias[i] = -1;
        return OMK_OK;
    }
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipStreamSynchronize(f->stream));
    HIP_TRY(hipMemcpy(h_alias, f->alias, (size_t)n_nodes * 4, hipMemcpyDeviceToHost));
    return OMK_OK;
}

int omk_tt_download_meta(omk_tt *tt, omk_tt_meta *h_meta) {
    if (!tt || !h_meta) return fail(OMK_ERR_INVALID, "omk_tt_download_meta: null argument");
    if (int rc = use_device(tt->f)) return rc;
    HIP_TRY(hipStreamSynchronize(tt->f->stream));
    static_assert(sizeof(omk_tt_meta) == sizeof(TTMeta), "the ABI struct mirrors the device one");
    HIP_TRY(hipMemcpy(h_meta, tt->meta, sizeof(TTMeta) << tt->log2_slots, hipMemcpyDeviceToHost));
    return OMK_OK;
}

int omk_batch_leaf_keys(omk_batch *b, const uint64_t *d_piece_keys, int32_t cells, const uint64_t *d_player_keys,
                        const uint64_t *d_root_keys, const int32_t *d_root_players, uint64_t *d_out) {
    if (!b || !d_piece_keys || !d_player_keys || !d_root_keys || !d_root_players || !d_out)
        return fail(OMK_ERR_INVALID, "omk_batch_leaf_keys: null argument");
    if (cells <= 0) return fail(OMK_ERR_INVALID, "omk_batch_leaf_keys: cells %d", cells);
    if (!b->selected) return fail(OMK_ERR_STATE, "omk_batch_leaf_keys: no selected paths");
    if (int rc = fresh_batch("omk_batch_leaf_keys", b)) return rc;
    omk_forest *f = b->f;
    if (int rc = use_device(f)) return rc;
    hipStream_t s = f->stream;
    int32_t *d_status = b->counters + 32;  // a word of the batch's counter block that nothing else uses
    int bad = 0;
    HIP_TRY(hipMemcpyAsync(d_status, &bad, sizeof(bad), hipMemcpyHostToDevice, s));
    HIP_TRY(launch_leaf_keys(f->dev(), b->paths, b->path_len, b->n, b->stride, d_piece_keys, cells, d_player_keys,
                             d_root_keys, d_root_players, d_out, d_status, s));
    HIP_TRY(hipMemcpyAsync(&bad, d_status, sizeof(bad), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    if (bad)
        return fail(OMK_ERR_INVALID, "omk_batch_leaf_keys: %d paths hold a move outside [0, %d) or no node at all "
                    "(their keys are ~0)", bad, cells);
    return OMK_OK;
}

int omk_tt_upload(omk_tt *tt, const omk_tt_slot *h_slots) {
    if (!tt || !h_slots) return fail(OMK_ERR_INVALID, "omk_tt_upload: null argument");
    if (int rc = use_device(tt->f)) return rc;
    HIP_TRY(hipStreamSynchronize(tt->f->stream));
    HIP_TRY(hipMemcpy(tt->slots, h_slots, sizeof(TTSlot) << tt->log2_slots, hipMemcpyHostToDevice));
    tt->generation = tt->f->generation;  // the caller's node ids are ids of the forest as it is now
    return OMK_OK;
}

int omk_tt_download(omk_tt *tt, omk_tt_slot *h_slots) {
    if (!tt || !h_slots) return fail(OMK_ERR_INVALID, "omk_tt_download: null argument");
    if (int rc = use_device(tt->f)) return rc;
    HIP_TRY(hipStreamSynchronize(tt->f->stream));
    HIP_TRY(hipMemcpy(h_slots, tt->slots, sizeof(TTSlot) << tt->log2_slots, hipMemcpyDeviceToHost));
    return OMK_OK;
}

// ---------------------------------------------------------------- device memory helpers

int omk_dev_alloc(omk_forest *f, int64_t bytes, void **d_out) {
    if (!f || !d_out || bytes < 0) return fail(OMK_ERR_INVALID, "omk_dev_alloc: bad argument");
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipMalloc(d_out, (size_t)std::max<int64_t>(bytes, 1)));
    return OMK_OK;
}

int omk_dev_free(omk_forest *f, void *d_ptr) {
    if (!f) return fail(OMK_ERR_INVALID, "omk_dev_free: null forest");
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipStreamSynchronize(f->stream));
    if (d_ptr) HIP_TRY(hipFree(d_ptr));
    return OMK_OK;
}

int omk_dev_copy(omk_forest *f, void *d_dst, const void *d_src, int64_t bytes) {
    if (!f || !d_dst || !d_src || bytes < 0 || (bytes & 3)) return fail(OMK_ERR_INVALID, "omk_dev_copy: bad argument");
    if (int rc = use_device(f)) return rc;
    HIP_TRY(launch_copy_words(d_dst, d_src, bytes / 4, f->stream));
    return OMK_OK;
}

int omk_dev_h2d(omk_forest *f, void *d_dst, const void *h_src, int64_t bytes) {
    if (!f || !d_dst || !h_src || bytes < 0) return fail(OMK_ERR_INVALID, "omk_dev_h2d: bad argument");
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipMemcpyAsync(d_dst, h_src, (size_t)bytes, hipMemcpyHostToDevice, f->stream));
    HIP_TRY(hipStreamSynchronize(f->stream));
    return OMK_OK;
}

int omk_dev_d2h(omk_forest *f, void *h_dst, const void *d_src, int64_t bytes) {
    if (!f || !h_dst || !d_src || bytes < 0) return fail(OMK_ERR_INVALID, "omk_dev_d2h: bad argument");
    if (int rc = use_device(f)) return rc;
    HIP_TRY(hipMemcpyAsync(h_dst, d_src, (size_t)bytes, hipMemcpyDeviceToHost, f->stream));
    HIP_TRY(hipStreamSynchronize(f->stream));
    return OMK_OK;
}

}  // extern "C"
