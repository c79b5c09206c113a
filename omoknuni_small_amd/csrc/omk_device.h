// Device-side building blocks shared by the kernels: wave64 cross-lane reductions
// written with DPP row operations, the order-preserving score key and the per-child
// score arithmetic of MCTSNode::selectChild (reference src/mcts/mcts_node.cpp:94-95,
// 143-160, 196-214) and getCombinedValue (:657-678).
//
// Everything here assumes all 64 lanes of the wavefront are active at the call site.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

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

// Maps a score to an unsigned key with the same order as the float comparison used by
// "score > best_score" (mcts_node.cpp:163,216).  A score that can never beat the initial
// -infinity (NaN or -infinity itself) maps to 0, below every real key.
__device__ __forceinline__ uint32_t score_key(float s) {
    if (!(s > -__builtin_inff())) return 0u;
    s = s + 0.0f;  // -0.0 and +0.0 compare equal: give them one key
    uint32_t b = __float_as_uint(s);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__device__ __forceinline__ float combined_value(int visits, float w, int rave_visits, float rw, float rave_k) {
    if (visits == 0 && rave_visits == 0) return 0.0f;
    float mcts_value = visits > 0 ? w / (float)visits : 0.0f;
    float rave_value = rave_visits > 0 ? rw / (float)rave_visits : 0.0f;
    int three_v = (int)(3u * (uint32_t)visits);
    float beta = sqrtf(rave_k / ((float)three_v + rave_k));
    float a = (1.0f - beta) * mcts_value;
    float b = beta * rave_value;
    return a + b;
}

// Keys of the two candidates a child contributes: its score in the first scan of
// selectChild and its score in the second scan.  The second differs from the first only
// through the RAVE blend q2 (getCombinedValue: it does not depend on virtual loss, so the
// caller computes it once per child) or, without RAVE, when 1 + ev is not exact in
// binary32; a second score equal to the first can never win (strict comparison, first
// scan comes first), so it is reported as 0.  While |ev| < 2^24 the divisors 1.0f + ev
// (first scan) and float(1 + ev) (second scan) are the same number, so one division
// serves both.
template <bool RAVE>
__device__ __forceinline__ void child_keys(int n, float w, float p, int vl, float q2, float ep, uint32_t &k1,
                                           uint32_t &k2) {
    int ev = (int)((uint32_t)n + (uint32_t)vl);
    float evalue = w - (float)vl;
    float q = ev > 0 ? evalue / (float)ev : 0.0f;
    float prod = p * ep;
    float u1 = prod / (1.0f + (float)ev);
    k1 = score_key(q + u1);
    const bool exact = ev < (1 << 24) && ev > -(1 << 24);
    if (RAVE) {
        float u2 = u1;
        if (!exact) u2 = prod / (float)(int)(1u + (uint32_t)ev);
        k2 = score_key(q2 + u2);
    } else if (!exact) {
        float u2 = prod / (float)(int)(1u + (uint32_t)ev);
        k2 = score_key(q + u2);
    } else {
        k2 = 0u;
    }
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
