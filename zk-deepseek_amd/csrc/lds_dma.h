// Helpers shared by the kernels that stream raw operand elements through LDS rings: loads that bypass the registers
// (global_load_lds_dwordx4), waits by count, and the digit split of a fragment of 16 elements held by one lane.
#pragma once
#include "gemm_mfma_kernels.h"

namespace zk {

// ---- loads that bypass the registers ------------------------------------------------------------------------
// global_load_lds_dwordx4 moves 16 bytes per lane from global memory straight into LDS: one wave-instruction fills
// 1 KB at a wave-uniform base (M0), lane l at byte 16 l.  The compiler does not know that these instructions load or
// that they write LDS, so the waits are explicit: vector-memory loads of a wave complete in order, and "at most N
// outstanding" with N = the loads issued since guarantees that everything older has landed.
__device__ __forceinline__ void lds_dma16(const void *gptr, unsigned lds_base)
{
    // (the base is the same in every lane, but derived from the wavefront's number, which the compiler holds in a vector register)
    // M0 is put back as it was: the compiler does not see the statement write it (the register cannot be named as
    // clobbered) and may be keeping a value of its own there across the statement.
    unsigned saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0) : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(gptr) : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));      // expcnt and lgkmcnt left at their maxima
}

// ---- digit split of a fragment (16 elements of one row) ----------------------------------------------------
// 64-bit elements, any digit count: two groups of 8, k ascending within the fragment
template <int N>
__device__ __forceinline__ void split16(const int64_t (&x)[16], v4i (&out)[N])
{
    uint2 a[N], b[N];
    limb_split8<N>(*reinterpret_cast<const int64_t(*)[8]>(&x[0]), a);
    limb_split8<N>(*reinterpret_cast<const int64_t(*)[8]>(&x[8]), b);
#pragma unroll
    for (int i = 0; i < N; i++) out[i] = v4i{ (int)a[i].x, (int)a[i].y, (int)b[i].x, (int)b[i].y };
}

// Elements that fit 32 bits.  N <= 4: x + bias stays inside 32 bits (the caller has checked |x| < 2^(8N-2)), the digits
// are its bytes.  N == 5 (any int32): the fifth digit is the carry of the biased sum of a non-negative element.
template <int N>
__device__ __forceinline__ void split16_w32(const int (&x)[16], v4i (&out)[N])
{
    constexpr uint32_t bias = N >= 5 ? 0x80808080u : (0x00808080u >> (8 * (4 - N)));
#pragma unroll
    for (int w = 0; w < 4; w++) {
        uint32_t y[4], o[4], e = 0;
#pragma unroll
        for (int z = 0; z < 4; z++) {
            const uint32_t xv = (uint32_t)x[4 * w + z], u = xv + bias;
            if (N >= 5) e |= ((u < bias && x[4 * w + z] >= 0) ? 1u : 0u) << (8 * z);
            y[z] = u ^ bias;
        }
        transpose4(y[0], y[1], y[2], y[3], o);
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (i < N) out[i][w] = (int)o[i];
        if (N >= 5) out[4][w] = (int)e;
    }
}

}  // namespace zk
