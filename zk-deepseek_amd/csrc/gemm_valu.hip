// GEMM path (a): native 64-bit multiply-add chains on the vector ALU.
//
// A 64x64 output tile per 256-thread workgroup, 4x4 outputs per thread, every output accumulated in a
// full 128-bit register quad (the reference's __int128 sum, inference/int64_gemm.cu:21-27).  Operand
// tiles of 16 k-steps are staged through LDS transposed to [k][row] so the inner loop reads 32-byte
// vectors; global loads are 128-byte row segments.  Handles every descriptor: int32 or int64 B, either B
// layout, operand divisors, any shape.
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
};

template <bool B32>
__device__ __forceinline__ int64_t load_b(const void *B, long off)
{
    return B32 ? (int64_t)reinterpret_cast<const int32_t *>(B)[off] : reinterpret_cast<const int64_t *>(B)[off];
}

template <bool B32, bool KMAJOR, bool RESCALE>
__global__ __launch_bounds__(256) void gemm_valu_kernel(ValuParams p)
{
    __shared__ int64_t As[kVK][kVP];
    __shared__ int64_t Bs[kVK][kVP];

    const int tid = threadIdx.x;
    const int g = blockIdx.z;
    const int m0 = blockIdx.y * kVT, n0 = blockIdx.x * kVT;
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
            ra[i] = RESCALE ? tdiv64(v, p.a_rs) : v;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int n, k;
            if (KMAJOR) { n = n0 + ln + i; k = k0 + kk_b; }
            else { n = n0 + lrow; k = k0 + lk + i; }
            int64_t v = (n < p.N && k < p.K) ? load_b<B32>(p.B, boff + (long)n * p.ldbn + (long)k * p.ldbk) : 0;
            rb[i] = RESCALE ? tdiv64(v, p.b_rs) : v;
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

template <bool B32, bool KMAJOR>
static void launch2(const ValuParams &p, dim3 grid, bool rescale)
{
    if (rescale) gemm_valu_kernel<B32, KMAJOR, true><<<grid, dim3(256), 0, 0>>>(p);
    else gemm_valu_kernel<B32, KMAJOR, false><<<grid, dim3(256), 0, 0>>>(p);
}

void gemm_valu_launch(const GemmDesc &d)
{
    ValuParams p;
    p.A = d.A; p.B = d.B; p.C = d.C; p.R = d.R;
    p.lda = d.lda; p.sA = d.sA; p.ldbn = d.ldbn; p.ldbk = d.ldbk; p.sB = d.sB; p.ldc = d.ldc; p.sC = d.sC;
    p.M = d.M; p.N = d.N; p.K = d.K; p.shift = d.shift;
    p.init = d.init; p.a_rs = d.a_rs; p.b_rs = d.b_rs;
    const bool rescale = d.a_rs != 1 || d.b_rs != 1;
    const bool kmajor = d.ldbn == 1 && d.ldbk != 1;
    const int gy_total = (d.M + kVT - 1) / kVT;
    const int gx = (d.N + kVT - 1) / kVT;
    // grid.y and grid.z are limited to 65535: walk M and G in chunks when they are larger
    for (int g0 = 0; g0 < d.G; g0 += 65535) {
        int gz = d.G - g0 < 65535 ? d.G - g0 : 65535;
        for (int y0 = 0; y0 < gy_total; y0 += 65535) {
            int gy = gy_total - y0 < 65535 ? gy_total - y0 : 65535;
            ValuParams q = p;
            q.A = p.A + (long)g0 * p.sA + (long)y0 * kVT * p.lda;
            q.B = d.b32 ? (const void *)((const int32_t *)p.B + (long)g0 * p.sB)
                        : (const void *)((const int64_t *)p.B + (long)g0 * p.sB);
            q.C = p.C + (long)g0 * p.sC + (long)y0 * kVT * p.ldc;
            q.R = p.R ? p.R + (long)g0 * p.sC + (long)y0 * kVT * p.ldc : nullptr;
            q.M = d.M - y0 * kVT;
            dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)gz);
            if (d.b32) { if (kmajor) launch2<true, true>(q, grid, rescale); else launch2<true, false>(q, grid, rescale); }
            else { if (kmajor) launch2<false, true>(q, grid, rescale); else launch2<false, false>(q, grid, rescale); }
        }
    }
}

}  // namespace zk
