// Breadth-first renumbering of a subtree on the device, for the compaction that follows
// re-rooting (tree reuse between moves: MCTSEngine::searchWithTreeReuse,
// reference src/mcts/mcts_engine_search.cpp:1029-1075, keeps the subtree of the move played
// and drops the rest; with arrays instead of pointers the kept nodes are renumbered so that
// siblings stay contiguous).
//
// order[] receives the old id of every new node: new id 0 is the new root, then level after
// level, a level in the order of its parents, the children of a parent in slot order.  One
// level at a time: the child counts of the level's nodes, an exclusive scan over them
// (rocPRIM through hipCUB) that gives every node the place of its first child in the next
// level, and one kernel that writes the children's old ids there.  new_begin[] receives the
// new id of every node's first child (0 for a node without children).
#include <hipcub/hipcub.hpp>

#include "omk_internal.h"

namespace omk {

__global__ __launch_bounds__(256) void k_bfs_counts(const int2 *span, const int32_t *order, int64_t lo, int64_t cnt,
                                                    int32_t *cc) {
    const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p < cnt) {
        const int c = span[order[lo + p]].y;
        cc[p] = c > 0 ? c : 0;
    }
}

// One wavefront per node of the level: its children's old ids go to the next level.
__global__ __launch_bounds__(256) void k_bfs_expand(const int2 *span, int32_t *order, int32_t *new_begin, int64_t lo,
                                                    int64_t cnt, int64_t next_lo, const int32_t *scan) {
    const int64_t p = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (p >= cnt) return;
    const int2 sp = span[order[lo + p]];
    const int64_t first = next_lo + scan[p];
    if (lane == 0) new_begin[lo + p] = sp.y > 0 ? (int32_t)first : 0;
    for (int j = lane; j < sp.y; j += 64) order[first + j] = sp.x + j;
}

// legal bit of new node i = legal bit of old node order[i]; one thread per word of the new mask
__global__ __launch_bounds__(256) void k_gather_legal(uint32_t *dst, const uint32_t *src, const int32_t *order,
                                                      int64_t k) {
    const int64_t w = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (w * 32 >= k) return;
    uint32_t word = 0u;
    for (int b = 0; b < 32 && w * 32 + b < k; b++) {
        const uint32_t old = (uint32_t)order[w * 32 + b];
        word |= ((src[old >> 5] >> (old & 31u)) & 1u) << b;
    }
    dst[w] = word;
}

// Plain fill kernel: used instead of hipMemsetAsync wherever a caller might capture the stream
// into a graph.
__global__ __launch_bounds__(256) void k_fill_words(uint32_t *dst, uint32_t value, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * 256;
    for (; i < n; i += step) dst[i] = value;
}

hipError_t launch_fill_words(void *dst, uint32_t value, int64_t n_words, hipStream_t s) {
    if (n_words <= 0) return hipSuccess;
    int64_t blocks = (n_words + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(k_fill_words, dim3((unsigned)blocks), dim3(256), 0, s, (uint32_t *)dst, value, n_words);
    return hipGetLastError();
}

hipError_t bfs_scan_bytes(int64_t max_items, size_t *bytes) {
    *bytes = 0;
    return hipcub::DeviceScan::ExclusiveSum(nullptr, *bytes, (const int32_t *)nullptr, (int32_t *)nullptr,
                                            (int)max_items, (hipStream_t)0);
}

// One level: nodes order[lo .. lo+cnt).  h_total receives the number of their children
// (the size of the next level, which starts at lo + cnt); waits for the stream.
hipError_t launch_bfs_level(const int2 *span, int32_t *order, int32_t *new_begin, int64_t lo, int64_t cnt,
                            int64_t room, int32_t *cc, int32_t *scan, void *temp, size_t temp_bytes,
                            int64_t *h_total, hipStream_t s) {
    hipLaunchKernelGGL(k_bfs_counts, dim3((unsigned)((cnt + 255) / 256)), dim3(256), 0, s, span, order, lo, cnt, cc);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    e = hipcub::DeviceScan::ExclusiveSum(temp, temp_bytes, (const int32_t *)cc, scan, (int)cnt, s);
    if (e != hipSuccess) return e;
    int32_t last[2] = {0, 0};
    e = hipMemcpyAsync(&last[0], scan + cnt - 1, 4, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipMemcpyAsync(&last[1], cc + cnt - 1, 4, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) return e;
    *h_total = (int64_t)last[0] + last[1];
    if (*h_total > room) return hipSuccess;  // the caller reports it: the child ranges do not form a tree
    if (*h_total > 0) {
        hipLaunchKernelGGL(k_bfs_expand, dim3((unsigned)((cnt + 3) / 4)), dim3(256), 0, s, span, order, new_begin, lo,
                           cnt, lo + cnt, scan);
        e = hipGetLastError();
    } else {
        e = launch_fill_words(new_begin + lo, 0u, cnt, s);
    }
    return e;
}

hipError_t launch_gather_legal(uint32_t *dst, const uint32_t *src, const int32_t *order, int64_t k, hipStream_t s) {
    if (k <= 0) return hipSuccess;
    const int64_t words = (k + 31) / 32;
    hipLaunchKernelGGL(k_gather_legal, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, s, dst, src, order, k);
    return hipGetLastError();
}

}  // namespace omk
