// One element of the fixed-point sigmoid / SiLU, shared by the streaming kernels and the gate's fused routing.
#pragma once
#include "common.h"

namespace zk {

// sigma(x) = 1 / (1 + e^-x) with e^-x = 2^y, y = -x*log2(e) split into an integer part k (a shift) and a fraction
// looked up in a 256-entry table; the reciprocal is an exact integer divide.
// Follows inference/int64_gemm.cu:903-947, :969-1017 (Q23) and :775-819, :841-882 (Q25).
template <int Q> struct ActConst;
template <> struct ActConst<23> { static constexpr int64_t kLog2e = 12102203; };
template <> struct ActConst<25> { static constexpr int64_t kLog2e = 48408813; };

template <int Q, bool SIGMOID>
__device__ __forceinline__ int64_t act_one(int64_t r, const int64_t *lut)
{
    constexpr int64_t LIM = (int64_t)64 << Q;
    constexpr int64_t ONE = (int64_t)1 << Q;
    if (r >= LIM) return r;     // the sigmoid kernels return x here as well
    if (r <= -LIM) return 0;
    // |r| < 2^(Q+6) and log2(e)*2^Q < 2^(Q+1): the product needs 2Q+8 <= 58 bits, so int64 is exact.
    int64_t y;
    if (Q == 23) y = ((-r) * ActConst<Q>::kLog2e) >> Q;    // negate, multiply, shift
    else y = -((r * ActConst<Q>::kLog2e) >> Q);             // multiply, shift, negate
    int64_t k = y >> Q;
    int64_t f = y & (ONE - 1);
    int64_t t = lut[f >> (Q - 8)];
    int64_t u = 0;
    if (k > -63) {
        if (k < 0) u = t >> (int)(-k);
        else u = (k >= 64) ? 0 : (int64_t)((uint64_t)t << (int)k);    // shifts of 64 or more give 0
    }
    int64_t den = (int64_t)((uint64_t)ONE + (uint64_t)u);
    int64_t q;
    if (den >= ONE && den < ((int64_t)1 << 53)) {
        constexpr uint64_t NUM = (uint64_t)1 << (2 * Q);
        q = (int64_t)udiv_by_inv(NUM, (uint64_t)den, 1.0 / (double)den);
    } else {
        q = tdiv64((int64_t)1 << (2 * Q), den);
    }
    if (SIGMOID) return q;
    return (int64_t)((uint64_t)r * (uint64_t)q) >> Q;
}

}  // namespace zk
