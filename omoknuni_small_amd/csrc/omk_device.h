// Device-side building blocks shared by the kernels: wave64 cross-lane reductions
// written with DPP row operations, the order-preserving score key and the per-child
// score arithmetic of MCTSNode::selectChild (reference src/mcts/mcts_node.cpp:94-95,
// 143-160, 196-214) and getCombinedValue (:657-678).
//
// Everything here assumes all 64 lanes of the wavefront are active at the call site.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "omk_score.h"

namespace omk {

constexpr int kWave = 64;

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_mov(uint32_t v) {
    // lanes whose source lane does not exist keep their own value
    return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xF, 0xF, false);
}

__device__ __forceinline__ uint32_t umax32(uint32_t a, uint32_t b) { return a > b ? a : b; }
__device__ __forceinline__ uint32_t umin32(uint32_t a, uint32_t b) { return a < b ? a : b; }

// Butterfly inside each row of 16 lanes (quad swaps, then row shifts by 4 and 8), after
// which lane 15 of every row holds the row's result; the four row results are combined
// on the scalar unit.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    v = umax32(v, dpp_mov<0xB1>(v));   // quad_perm [1,0,3,2]
    v = umax32(v, dpp_mov<0x4E>(v));   // quad_perm [2,3,0,1]
    v = umax32(v, dpp_mov<0x114>(v));  // row_shr:4
    v = umax32(v, dpp_mov<0x118>(v));  // row_shr:8
    uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 15);
    uint32_t b = (uint32_t)__builtin_amdgcn_readlane((int)v, 31);
    uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 47);
    uint32_t d = (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
    return umax32(umax32(a, b), umax32(c, d));
}

__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
    v = umin32(v, dpp_mov<0xB1>(v));
    v = umin32(v, dpp_mov<0x4E>(v));
    v = umin32(v, dpp_mov<0x114>(v));
    v = umin32(v, dpp_mov<0x118>(v));
    uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 15);
    uint32_t b = (uint32_t)__builtin_amdgcn_readlane((int)v, 31);
    uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 47);
    uint32_t d = (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
    return umin32(umin32(a, b), umin32(c, d));
}

// Sum over the 64 lanes: xor butterfly inside each row of 16 (quad swaps, half-row mirror,
// row mirror leave the row total in every lane), the four row totals added on the scalar unit.
__device__ __forceinline__ int wave_sum_i32(int x) {
    uint32_t v = (uint32_t)x;
    v += dpp_mov<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_mov<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_mov<0x141>(v);  // row_half_mirror
    v += dpp_mov<0x140>(v);  // row_mirror
    uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0);
    uint32_t b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32);
    uint32_t d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    return (int)(a + b + c + d);
}

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_mov_zero(uint32_t v) {
    // lanes whose source lane does not exist receive 0
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}

// Inclusive prefix sum over the 64 lanes: log-step scan inside each row of 16 with row
// shifts, then the totals of the rows below are added from the scalar unit.
__device__ __forceinline__ int wave_inclusive_sum(int x, int lane) {
    uint32_t v = (uint32_t)x;
    v += dpp_mov_zero<0x111>(v);  // row_shr:1
    v += dpp_mov_zero<0x112>(v);  // row_shr:2
    v += dpp_mov_zero<0x114>(v);  // row_shr:4
    v += dpp_mov_zero<0x118>(v);  // row_shr:8
    uint32_t t0 = (uint32_t)__builtin_amdgcn_readlane((int)v, 15);
    uint32_t t1 = (uint32_t)__builtin_amdgcn_readlane((int)v, 31);
    uint32_t t2 = (uint32_t)__builtin_amdgcn_readlane((int)v, 47);
    const int row = lane >> 4;
    uint32_t add = row >= 1 ? t0 : 0u;
    add += row >= 2 ? t1 : 0u;
    add += row >= 3 ? t2 : 0u;
    return (int)(v + add);
}

__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) v += __shfl_xor(v, d, kWave);
    return v;
}

// smallest k >= 1 with k*k >= n
__device__ __forceinline__ int ceil_sqrt_i32(int n) {
    if (n <= 1) return 1;
    long long k = (long long)sqrt((double)n);
    while (k * k < (long long)n) k++;
    while ((k - 1) * (k - 1) >= (long long)n) k--;
    return (int)k;
}

}  // namespace omk
