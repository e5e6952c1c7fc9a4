// GEMM path (a): native 64-bit multiply-add chains on the vector ALU.
//
// A 64x64 output tile per 256-thread workgroup, 4x4 outputs per thread, every output accumulated in a
// full 128-bit register quad (the reference's __int128 sum, inference/int64_gemm.cu:21-27).  Operand
// tiles of 16 k-steps are staged through LDS transposed to [k][row] so the inner loop reads 32-byte
// vectors; global loads are 128-byte row segments.  Handles every descriptor: int32 or int64 B, either B
// layout, operand divisors, any shape.
//
// The same kernel is the safety net of the speculating MFMA path: launched with a `guard` word, its workgroups
// return at once unless that word says the speculation failed, in which case they recompute every output.
#include "gemm.h"

namespace zk {

constexpr int kVT = 64;        // tile edge (rows of A and of B per workgroup)
constexpr int kVK = 16;        // k-steps per LDS stage
constexpr int kVP = 68;        // padded row length of the [k][row] LDS tiles (int64 units)

struct ValuParams {
    const int64_t *A;
    const void *B;
    int64_t *C, *R;
    long lda, sA, ldbn, ldbk, sB, ldc, sC;
    int M, N, K, shift;
    int64_t init, a_rs, b_rs;
    int a_shift, b_shift;                     // log2 of a divisor that is a positive power of two, else -1
    int tiles_m, tiles_n;
    long tiles;                               // tiles_m * tiles_n * G, walked by a 1-D grid
    const unsigned long long *guard;          // when set: do nothing unless *guard != 0
};

template <bool B32>
__device__ __forceinline__ int64_t load_b(const void *B, long off)
{
    return B32 ? (int64_t)reinterpret_cast<const int32_t *>(B)[off] : reinterpret_cast<const int64_t *>(B)[off];
}

// operand / divisor as C++ computes it; divisors that are powers of two (the model's only ones: 1 and 256) are shifts
__device__ __forceinline__ int64_t rescale_operand(int64_t v, int64_t rs, int shift)
{
    if (shift >= 0) {
        const uint64_t bias = (uint64_t)(v >> 63) & (((uint64_t)1 << shift) - 1);
        return (int64_t)((uint64_t)v + bias) >> shift;
    }
    return tdiv64(v, rs);
}

template <bool B32, bool KMAJOR, bool RESCALE>
__global__ __launch_bounds__(256) void gemm_valu_kernel(ValuParams p)
{
    __shared__ int64_t As[kVK][kVP];
    __shared__ int64_t Bs[kVK][kVP];

    const int tid = threadIdx.x;
    if (p.guard && __atomic_load_n(p.guard, __ATOMIC_RELAXED) == 0) return;
    for (long tile = blockIdx.x; tile < p.tiles; tile += gridDim.x) {
    const int g = (int)(tile / ((long)p.tiles_m * p.tiles_n));
    const int rem = (int)(tile - (long)g * p.tiles_m * p.tiles_n);
    const int m0 = (rem / p.tiles_n) * kVT, n0 = (rem % p.tiles_n) * kVT;
    const int64_t *Ag = p.A + (long)g * p.sA;
    const long boff = (long)g * p.sB;

    // loader coordinates: A and n-major B read 4 consecutive k of one row; k-major B reads 4 consecutive n of one k
    const int lrow = tid >> 2, lk = (tid & 3) * 4;
    const int kk_b = tid >> 4, ln = (tid & 15) * 4;

    u128 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = 0;

    const int ty = tid >> 4, tx = tid & 15;
    int64_t ra[4], rb[4];

    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int m = m0 + lrow, k = k0 + lk + i;
            int64_t v = (m < p.M && k < p.K) ? Ag[(long)m * p.lda + k] : 0;
            ra[i] = RESCALE ? rescale_operand(v, p.a_rs, p.a_shift) : v;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int n, k;
            if (KMAJOR) { n = n0 + ln + i; k = k0 + kk_b; }
            else { n = n0 + lrow; k = k0 + lk + i; }
            int64_t v = (n < p.N && k < p.K) ? load_b<B32>(p.B, boff + (long)n * p.ldbn + (long)k * p.ldbk) : 0;
            rb[i] = RESCALE ? rescale_operand(v, p.b_rs, p.b_shift) : v;
        }
    };

    fetch(0);
    for (int k0 = 0; k0 < p.K; k0 += kVK) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            As[lk + i][lrow] = ra[i];
            if (KMAJOR) Bs[kk_b][ln + i] = rb[i];
            else Bs[lk + i][lrow] = rb[i];
        }
        __syncthreads();
        if (k0 + kVK < p.K) fetch(k0 + kVK);
#pragma unroll
        for (int kk = 0; kk < kVK; kk++) {
            int64_t a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; i++) { a[i] = As[kk][ty * 4 + i]; b[i] = Bs[kk][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] += (u128)((i128)a[i] * (i128)b[j]);
        }
        __syncthreads();
    }

    const uint64_t rmask = p.shift ? ((1ull << p.shift) - 1) : 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int m = m0 + ty * 4 + i;
        if (m >= p.M) continue;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int n = n0 + tx * 4 + j;
            if (n >= p.N) continue;
            u128 sum = acc[i][j] + (u128)(i128)p.init;
            long o = (long)g * p.sC + (long)m * p.ldc + n;
            p.C[o] = (int64_t)(uint64_t)((i128)sum >> p.shift);
            if (p.R) p.R[o] = (int64_t)((uint64_t)sum & rmask);
        }
    }
    }
}

template <bool B32, bool KMAJOR>
static void launch2(const ValuParams &p, dim3 grid, bool rescale)
{
    if (rescale) gemm_valu_kernel<B32, KMAJOR, true><<<grid, dim3(256), 0, 0>>>(p);
    else gemm_valu_kernel<B32, KMAJOR, false><<<grid, dim3(256), 0, 0>>>(p);
}

void gemm_valu_launch(const GemmDesc &d, const unsigned long long *guard)
{
    ValuParams p;
    p.A = d.A; p.B = d.B; p.C = d.C; p.R = d.R;
    p.lda = d.lda; p.sA = d.sA; p.ldbn = d.ldbn; p.ldbk = d.ldbk; p.sB = d.sB; p.ldc = d.ldc; p.sC = d.sC;
    p.M = d.M; p.N = d.N; p.K = d.K; p.shift = d.shift;
    p.init = d.init; p.a_rs = d.a_rs; p.b_rs = d.b_rs;
    auto log2_exact = [](int64_t v) {
        if (v <= 0 || (v & (v - 1)) != 0) return -1;
        int s = 0;
        while (((int64_t)1 << s) < v) s++;
        return s;
    };
    p.a_shift = log2_exact(d.a_rs);
    p.b_shift = log2_exact(d.b_rs);
    p.tiles_m = (d.M + kVT - 1) / kVT;
    p.tiles_n = (d.N + kVT - 1) / kVT;
    p.tiles = (long)p.tiles_m * p.tiles_n * d.G;
    p.guard = guard;
    const bool rescale = d.a_rs != 1 || d.b_rs != 1;
    const bool kmajor = d.ldbn == 1 && d.ldbk != 1;
    // a guarded launch normally finds nothing to do, so it is kept small; either way workgroups stride over the tiles
    const long cap = guard ? 2048 : (1L << 22);
    dim3 grid((unsigned)(p.tiles < cap ? p.tiles : cap));
    if (d.b32) { if (kmajor) launch2<true, true>(p, grid, rescale); else launch2<true, false>(p, grid, rescale); }
    else { if (kmajor) launch2<false, true>(p, grid, rescale); else launch2<false, false>(p, grid, rescale); }
}

}  // namespace zk
