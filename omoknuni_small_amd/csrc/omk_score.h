// The per-child score arithmetic of MCTSNode::selectChild (reference src/mcts/mcts_node.cpp:94-95,
// 143-160, 196-214) and getCombinedValue (:657-678), the order-preserving score key, and the
// test that proves a child's successive scores cannot increase.  Plain binary32 / binary64
// arithmetic without device builtins: compiled for the device by hipcc and for the host by any
// C++ compiler (tests check the proof test against brute force there).  Must be compiled without
// floating-point contraction, like everything that has to round as the reference does.
#pragma once

#include <math.h>
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define OMK_HD __host__ __device__ __forceinline__
#else
#define OMK_HD inline
#endif

namespace omk {

OMK_HD uint32_t omk_float_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, sizeof(u));
    return u;
}

// Maps a score to an unsigned key with the same order as the float comparison used by
// "score > best_score" (mcts_node.cpp:163,216).  A score that can never beat the initial
// -infinity (NaN or -infinity itself) maps to 0, below every real key.
OMK_HD uint32_t score_key(float s) {
    if (!(s > -__builtin_inff())) return 0u;
    s = s + 0.0f;  // -0.0 and +0.0 compare equal: give them one key
    uint32_t b = omk_float_bits(s);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

OMK_HD float combined_value(int visits, float w, int rave_visits, float rw, float rave_k) {
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
OMK_HD void child_keys(int n, float w, float p, int vl, float q2, float ep, uint32_t &k1,
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

// Sufficient test that the keys a child shows to its visits j = 0 .. j_last of one selection (its
// virtual loss at visit j is vl0 + j * uvl) do not increase, and that no later visit comes before an
// earlier one in the order (key descending, first-scan candidate before second-scan candidate):
// what the parallel paths otherwise check entry by entry.  The proof, step by step through
// child_keys, with x_j = n + vl_j the divisor and E_j = fl(w - vl_j) the rounded numerator:
//   * every x_j and 1 + x_j is below 2^24, so the conversions are exact and the second scan's
//     divisor equals the first's (child_keys' `exact` case; without RAVE the second key is 0);
//   * u_j = fl(prod / (1 + x_j)) with prod = fl(p * ep) >= 0 fixed: the real quotient falls as x
//     grows, and rounding keeps order;
//   * E_j does not increase (rounding keeps order).  While E_j >= 0: E_{j+1} <= E_j and
//     x_{j+1} > x_j > 0 give E_{j+1} / x_{j+1} <= E_j / x_j, rounded or not.  Where E_j < 0 that
//     needs E_{j+1} * x_j <= E_j * x_{j+1}; with E_j = w - vl_j + d_j, |d_j| <= 2^-24 |E_j|, it
//     reduces to uvl * (n + w) >= (d_{j+1} - d_j) * x_j - d_j * uvl, which
//     uvl * (n + w) >= 2^-23 * max|E| * (x_last + uvl) implies; when w is integral every E_j is
//     exact (d_j = 0) and n + w >= 0 suffices.  (n + w < 0, a value sum below minus the visit
//     count, makes the real quotient RISE with virtual loss: refused.)
//   * a child with x_0 = 0 scores q = 0 at visit 0 by definition; q_1 = fl(E_1 / x_1) <= 0 needs
//     w <= vl_1;
//   * sums of non-increasing terms, rounded, do not increase; score_key keeps order; the entry's key
//     is the larger of two non-increasing keys; an entry of the first scan cannot follow one of the
//     second scan at an EQUAL key (it would need k1_{j+1} = k2_j > k1_j >= k1_{j+1}).
// All inputs finite and in range, so no key is the "never selected" key 0 unless the first one is.
template <bool RAVE>
OMK_HD bool keys_provably_monotone(int n, float w, float p, int vl0, float q2, float ep, uint32_t uvl, int j_last) {
    if (n < 0 || vl0 < 0 || j_last < 0 || uvl == 0u || uvl > 1024u) return false;
    const double x_last = (double)n + (double)vl0 + (double)j_last * (double)uvl;
    if (!(x_last + 1.0 < 16777216.0)) return false;
    const float prod = p * ep;
    if (!(prod >= 0.0f) || !(prod < 3.0e38f)) return false;
    if (!(w > -3.0e38f) || !(w < 3.0e38f)) return false;
    if (RAVE && (!(q2 > -3.0e38f) || !(q2 < 3.0e38f))) return false;
    const double dw = (double)w;
    const double vl_last = (double)vl0 + (double)j_last * (double)uvl;
    if (n + vl0 == 0 && j_last >= 1 && !(dw <= (double)vl0 + (double)uvl)) return false;
    if (dw >= vl_last) return true;  // the numerator never turns negative
    // an integral value sum (an unvisited child's 0 above all): w - vl_j is exact, d_j = 0, and
    // n + w >= 0 is all that is needed
    if (w == floorf(w) && w > -16777216.0f && w < 16777216.0f) return (double)n + dw >= 0.0;
    const double e0 = fabs(dw - (double)vl0), e1 = fabs(dw - vl_last);
    const double emax = e0 > e1 ? e0 : e1;
    const double lhs = (double)uvl * ((double)n + dw);
    const double rhs = 1.1920928955078125e-7 * 1.001 * emax * (x_last + (double)uvl) + 1e-30;
    return lhs >= rhs;
}

}  // namespace omk
