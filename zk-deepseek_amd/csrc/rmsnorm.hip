// Integer RMSNorm: rms[m] = isqrt((eps + sum_n a^2) / dim) exactly (the sum needs up to 140 bits), then
// C = floor(a * w / rms) with a 128-bit product.
//
// The reference computes the statistic on the host, one device->host sync per element
// (inference/kernel.py:477-494, :539-542) and applies it with inference/int64_gemm.cu:289-385.
// Here one workgroup owns one row: the row is read once into registers, squared and summed in 192-bit
// integers, reduced across the workgroup, square-rooted by one lane, and normalised from registers.
#include "common.h"
#include "../../include/int64gemm.h"

namespace zk {

// ---- 192-bit unsigned accumulator -------------------------------------------------------------
struct U192 { uint64_t w0, w1, w2; };

__device__ __forceinline__ void u192_add(U192 &a, const U192 &b)
{
    uint64_t s0 = a.w0 + b.w0;
    uint64_t c0 = s0 < a.w0;
    uint64_t s1 = a.w1 + b.w1;
    uint64_t c1 = s1 < a.w1;
    uint64_t s1b = s1 + c0;
    c1 += s1b < s1;
    a.w0 = s0;
    a.w1 = s1b;
    a.w2 = a.w2 + b.w2 + c1;
}

// Per-thread sum of squares with three multiplies per element: for m = |v| = hi * 2^32 + lo,
//   m^2 = lo*lo + 2^33 * lo*hi + 2^64 * hi*hi,
// and each of the three products is summed in its own 64-bit column with a carry counter; the columns are merged
// once per thread.  (The compiler's 128-bit square of a sign-extended value costs three times the multiplies.)
struct SquareSum {
    uint64_t ll = 0, lh = 0, hh = 0;
    uint32_t cll = 0, clh = 0, chh = 0;
    __device__ __forceinline__ void add(int64_t v)
    {
        const uint64_t m = v < 0 ? 0 - (uint64_t)v : (uint64_t)v;
        const uint32_t lo = (uint32_t)m, hi = (uint32_t)(m >> 32);
        uint64_t t = ll + (uint64_t)lo * lo;
        cll += t < ll;
        ll = t;
        t = lh + (uint64_t)lo * hi;
        clh += t < lh;
        lh = t;
        t = hh + (uint64_t)hi * hi;
        chh += t < hh;
        hh = t;
    }
    __device__ __forceinline__ U192 total() const
    {
        U192 r = { ll, cll, 0 };                                               // ll + 2^64 cll
        // (lh + 2^64 clh) * 2^33
        const U192 mid = { lh << 33, (lh >> 31) | ((uint64_t)clh << 33), (uint64_t)clh >> 31 };
        u192_add(r, mid);
        const U192 top = { 0, hh, chh };                                       // (hh + 2^64 chh) * 2^64
        u192_add(r, top);
        return r;
    }
};

__device__ __forceinline__ U192 wave_sum_u192(U192 a)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        U192 o;
        o.w0 = (uint64_t)__shfl_xor((long long)a.w0, off, kWave);
        o.w1 = (uint64_t)__shfl_xor((long long)a.w1, off, kWave);
        o.w2 = (uint64_t)__shfl_xor((long long)a.w2, off, kWave);
        u192_add(a, o);
    }
    return a;
}

// floor(x / d), d > 0.  32-bit divisors (every model shape) use schoolbook division on 32-bit digits.
__device__ U192 u192_div(U192 x, uint64_t d)
{
    U192 q;
    if (d <= 0xFFFFFFFFull) {
        uint32_t dig[6] = { (uint32_t)x.w0, (uint32_t)(x.w0 >> 32), (uint32_t)x.w1,
                            (uint32_t)(x.w1 >> 32), (uint32_t)x.w2, (uint32_t)(x.w2 >> 32) };
        uint32_t qd[6];
        uint64_t rem = 0;
#pragma unroll
        for (int i = 5; i >= 0; i--) {
            uint64_t cur = (rem << 32) | dig[i];
            qd[i] = (uint32_t)(cur / d);
            rem = cur % d;
        }
        q.w0 = qd[0] | ((uint64_t)qd[1] << 32);
        q.w1 = qd[2] | ((uint64_t)qd[3] << 32);
        q.w2 = qd[4] | ((uint64_t)qd[5] << 32);
    } else {
        u128 rem = 0, cur;
        cur = (rem << 64) | x.w2; q.w2 = (uint64_t)(cur / d); rem = cur % d;
        cur = (rem << 64) | x.w1; q.w1 = (uint64_t)(cur / d); rem = cur % d;
        cur = (rem << 64) | x.w0; q.w0 = (uint64_t)(cur / d); rem = cur % d;
    }
    return q;
}

__device__ __forceinline__ double u128_to_double(u128 x)
{
    return (double)(uint64_t)(x >> 64) * 18446744073709551616.0 + (double)(uint64_t)x;
}

// floor(sqrt(x)) for x < 2^126 (so the root is below 2^63).  A double estimate is corrected once with the
// residual and then walked to the exact root; the walk is at most a few steps.
__device__ uint64_t isqrt_u128(u128 x)
{
    if (x == 0) return 0;
    uint64_t r = (uint64_t)sqrt(u128_to_double(x));
    if (r > 0x7FFFFFFFFFFFFFFFull) r = 0x7FFFFFFFFFFFFFFFull;
    {
        u128 rr = (u128)r * r;
        double e = rr > x ? -u128_to_double(rr - x) : u128_to_double(x - rr);
        double delta = floor(e / (2.0 * (double)r + 1.0));
        int64_t di = (int64_t)delta;
        r = (uint64_t)((int64_t)r + di);
        if (r > 0x7FFFFFFFFFFFFFFFull) r = 0x7FFFFFFFFFFFFFFFull;
    }
    while ((u128)r * r > x) r--;
    while (true) {
        u128 e = x - (u128)r * r;
        if (e >= 2 * (u128)r + 1 && r < 0x7FFFFFFFFFFFFFFFull) r++;
        else break;
    }
    return r;
}

// rms from the reduced sum.  Returns 0 and flags overflow when (eps + sum) / dim does not fit 126 bits.
__device__ int64_t rms_finalize(U192 acc, int64_t eps, int64_t dim)
{
    U192 e = { (uint64_t)eps, 0, 0 };
    u192_add(acc, e);
    U192 q = u192_div(acc, (uint64_t)dim);
    if (q.w2 != 0 || (q.w1 >> 62) != 0) return 0;
    return (int64_t)isqrt_u128(((u128)q.w1 << 64) | q.w0);
}

// floor(a * w / r) as the reference computes it: C++ division of the 128-bit product, minus one when the
// remainder is negative (inference/int64_gemm.cu:314-322).  r == 0 gives 0.
__device__ __noinline__ int64_t rms_apply_slow(int64_t a, int64_t w, int64_t r)
{
    if (r == 0) return 0;
    i128 prod = (i128)a * (i128)w;
    i128 qq = prod / (i128)r;
    i128 rr = prod % (i128)r;
    if (rr < 0) qq -= 1;
    return (int64_t)(uint64_t)(u128)qq;
}

// Fast exact path for 0 < r < 2^62 and |quotient| < 2^49.  The quotient is estimated in double precision from
// the operands themselves: a, w and 1/r each carry a relative error of at most 2^-53 and so does each of the two
// products, so the estimate is off by less than 2^49 * 5 * 2^-53 < 0.32 and, rounded to nearest, lands within
// one of the floor.  The remainder, exact modulo 2^64, settles which; anything else takes the slow path.
// The rounding and the conversion to an integer are one addition: for |x| < 2^51 the low bits of
// x + 1.5 * 2^52 hold round(x) as a fixed-point number.
template <typename WT>
__device__ __forceinline__ int64_t rms_apply_one(int64_t a, WT w, int64_t r, double inv_r, bool fast_r)
{
    if (fast_r) {
        const double xd = (double)a * (double)w * inv_r;
        if (fabs(xd) < 562949953421312.0) {
            const double magic = 6755399441055744.0;
            int64_t q = __double_as_longlong(xd + magic) - __double_as_longlong(magic);
            const uint64_t plo = (uint64_t)a * (uint64_t)(int64_t)w;
            int64_t rem = (int64_t)(plo - (uint64_t)q * (uint64_t)r);
            if (rem < 0) { q--; rem += r; }
            else if (rem >= r) { q++; rem -= r; }
            if (rem >= 0 && rem < r) return q;
        }
    }
    return rms_apply_slow(a, (int64_t)w, r);
}

constexpr int kRmsThreads = 256;
#ifndef ZK_RMS_T8K
#define ZK_RMS_T8K 512
#define ZK_RMS_E8K 16
#endif

template <int THREADS>
__device__ __forceinline__ U192 block_sum_u192(U192 acc, U192 *red)
{
    acc = wave_sum_u192(acc);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) red[wave] = acc;
    __syncthreads();
    U192 tot = red[0];
#pragma unroll
    for (int w = 1; w < THREADS / 64; w++) u192_add(tot, red[w]);
    return tot;
}

// Statistic only: one workgroup per row, any N.
__global__ __launch_bounds__(kRmsThreads) void rms_stat_kernel(const int64_t *__restrict__ A, int64_t *__restrict__ rms,
                                                               int N, int64_t eps, int64_t dim)
{
    __shared__ U192 red[kRmsThreads / 64];
    const int64_t *a = A + (long)blockIdx.x * N;
    SquareSum sq;
    for (int i = threadIdx.x; i < N; i += kRmsThreads) sq.add(a[i]);
    U192 tot = block_sum_u192<kRmsThreads>(sq.total(), red);
    if (threadIdx.x == 0) rms[blockIdx.x] = rms_finalize(tot, eps, dim);
}

typedef int v4i_r __attribute__((ext_vector_type(4)));

// Normalisation only, rms given (the reference's rms_norm_32 / rms_norm_64 contract).  A workgroup covers
// 256 * kApplyEpt consecutive elements of one row; VEC: N is even and the rows are 16-byte aligned.
constexpr int kApplyEpt = 8;
template <typename WT, bool VEC>
__global__ __launch_bounds__(kRmsThreads) void rms_apply_kernel(const int64_t *__restrict__ A, const WT *__restrict__ W,
                                                                const int64_t *__restrict__ rms, int64_t *__restrict__ C,
                                                                int N)
{
    const long row = blockIdx.y;
    const int64_t r = rms[row];
    const bool fast_r = r > 0 && r < ((int64_t)1 << 62);
    const double inv_r = fast_r ? 1.0 / (double)r : 0.0;
    const int base = blockIdx.x * (kRmsThreads * kApplyEpt);
    const int64_t *a = A + row * N;
    int64_t *c = C + row * N;
    if (VEC) {
        v4i_r t[kApplyEpt / 2];
#pragma unroll
        for (int j = 0; j < kApplyEpt / 2; j++) {
            const int i = base + (j * kRmsThreads + threadIdx.x) * 2;
            if (i < N) t[j] = __builtin_nontemporal_load(reinterpret_cast<const v4i_r *>(a + i));
        }
#pragma unroll
        for (int j = 0; j < kApplyEpt / 2; j++) {
            const int i = base + (j * kRmsThreads + threadIdx.x) * 2;
            if (i < N) {
                const int64_t v0 = (int64_t)(((uint64_t)(uint32_t)t[j][1] << 32) | (uint32_t)t[j][0]);
                const int64_t v1 = (int64_t)(((uint64_t)(uint32_t)t[j][3] << 32) | (uint32_t)t[j][2]);
                const int64_t c0 = rms_apply_one(v0, W[i], r, inv_r, fast_r);
                const int64_t c1 = rms_apply_one(v1, W[i + 1], r, inv_r, fast_r);
                const v4i_r o = { (int)(uint32_t)c0, (int)(uint32_t)((uint64_t)c0 >> 32), (int)(uint32_t)c1,
                                  (int)(uint32_t)((uint64_t)c1 >> 32) };
                __builtin_nontemporal_store(o, reinterpret_cast<v4i_r *>(c + i));
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < kApplyEpt; j++) {
            const int i = base + j * kRmsThreads + threadIdx.x;
            if (i < N) c[i] = rms_apply_one(a[i], W[i], r, inv_r, fast_r);
        }
    }
}

// Statistic + normalisation, one workgroup of THREADS per row, the row kept in registers (N <= THREADS * EPT).
// Long rows get more threads rather than more elements per thread: fewer registers mean more rows in flight per
// compute unit, which is what hides the serial stretch (reduction, division, square root) in the middle.
// VEC: N is even and the rows are 16-byte aligned: elements are moved two at a time with streaming accesses.
template <typename WT, int THREADS, int EPT, bool VEC>
__global__ __launch_bounds__(THREADS) void rms_fused_kernel(const int64_t *__restrict__ A, const WT *__restrict__ W,
                                                                int64_t *__restrict__ rms, int64_t *__restrict__ C,
                                                                int N, int64_t eps, int64_t dim)
{
    __shared__ U192 red[THREADS / 64];
    __shared__ int64_t rms_s;
    const long row = blockIdx.x;
    const int64_t *a = A + row * N;
    int64_t v[EPT];
    SquareSum sq;
    if (VEC) {
#pragma unroll
        for (int j = 0; j < EPT / 2; j++) {
            const int i = (j * THREADS + threadIdx.x) * 2;
            if (i < N) {
                const v4i_r t = __builtin_nontemporal_load(reinterpret_cast<const v4i_r *>(a + i));
                v[2 * j] = (int64_t)(((uint64_t)(uint32_t)t[1] << 32) | (uint32_t)t[0]);
                v[2 * j + 1] = (int64_t)(((uint64_t)(uint32_t)t[3] << 32) | (uint32_t)t[2]);
                sq.add(v[2 * j]);
                sq.add(v[2 * j + 1]);
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < EPT; j++) {
            const int i = j * THREADS + threadIdx.x;
            if (i < N) { v[j] = a[i]; sq.add(v[j]); }
        }
    }
    U192 tot = block_sum_u192<THREADS>(sq.total(), red);
    if (threadIdx.x == 0) {
        int64_t r = rms_finalize(tot, eps, dim);
        rms_s = r;
        rms[row] = r;
    }
    __syncthreads();
    const int64_t r = rms_s;
    const bool fast_r = r > 0 && r < ((int64_t)1 << 62);
    const double inv_r = fast_r ? 1.0 / (double)r : 0.0;
    if (VEC) {
#pragma unroll
        for (int j = 0; j < EPT / 2; j++) {
            const int i = (j * THREADS + threadIdx.x) * 2;
            if (i < N) {
                const int64_t c0 = rms_apply_one(v[2 * j], W[i], r, inv_r, fast_r);
                const int64_t c1 = rms_apply_one(v[2 * j + 1], W[i + 1], r, inv_r, fast_r);
                const v4i_r t = { (int)(uint32_t)c0, (int)(uint32_t)((uint64_t)c0 >> 32), (int)(uint32_t)c1,
                                  (int)(uint32_t)((uint64_t)c1 >> 32) };
                __builtin_nontemporal_store(t, reinterpret_cast<v4i_r *>(C + row * N + i));
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < EPT; j++) {
            const int i = j * THREADS + threadIdx.x;
            if (i < N) C[row * N + i] = rms_apply_one(v[j], W[i], r, inv_r, fast_r);
        }
    }
}

static bool rms_args_ok(const char *name, const void *A, const void *W, const void *rms, const void *C, int M, int N)
{
    if (M < 0 || N < 0) { set_error(kBadArgument, "%s: negative dimension", name); return false; }
    if ((long)M * N == 0) return false;
    if (!A || !rms || (!W && C) || (W && !C)) { set_error(kBadArgument, "%s: null pointer", name); return false; }
    return true;
}

template <typename WT>
static void launch_apply(const char *name, const int64_t *A, const WT *W, const int64_t *rms, int64_t *C, int M, int N)
{
    if (!rms_args_ok(name, A, W, rms, C, M, N)) return;
    if (M > 65535) { set_error(kUnsupportedSize, "%s: more than 65535 rows", name); return; }
    const int per_wg = kRmsThreads * kApplyEpt;
    dim3 grid((unsigned)((N + per_wg - 1) / per_wg), (unsigned)M);
    const bool vec = N % 2 == 0 && (((uintptr_t)A | (uintptr_t)C) & 15) == 0;
    if (vec) rms_apply_kernel<WT, true><<<grid, dim3(kRmsThreads), 0, 0>>>(A, W, rms, C, N);
    else rms_apply_kernel<WT, false><<<grid, dim3(kRmsThreads), 0, 0>>>(A, W, rms, C, N);
    check_launch(name);
}

static bool stat_args_ok(const char *name, int64_t eps, int64_t dim)
{
    if (dim <= 0) { set_error(kBadArgument, "%s: dim must be positive", name); return false; }
    if (eps < 0) { set_error(kBadArgument, "%s: eps must be non-negative", name); return false; }
    return true;
}

template <typename WT>
static void launch_fused(const char *name, const int64_t *A, const WT *W, int64_t *rms, int64_t *C, int M, int N,
                         int64_t eps, int64_t dim)
{
    if (!rms_args_ok(name, A, W, rms, C, M, N) || !stat_args_ok(name, eps, dim)) return;
    const bool vec = N % 2 == 0 && (((uintptr_t)A | (uintptr_t)C) & 15) == 0;
    const dim3 grid((unsigned)M);
#define ZK_RMS_LAUNCH(THREADS, EPT)                                                                                   \
    do {                                                                                                              \
        if (vec) rms_fused_kernel<WT, THREADS, EPT, true><<<grid, dim3(THREADS), 0, 0>>>(A, W, rms, C, N, eps, dim);   \
        else rms_fused_kernel<WT, THREADS, EPT, false><<<grid, dim3(THREADS), 0, 0>>>(A, W, rms, C, N, eps, dim);      \
    } while (0)
    if (N <= 512) ZK_RMS_LAUNCH(256, 2);
    else if (N <= 2048) ZK_RMS_LAUNCH(256, 8);
    else if (N <= 4096) ZK_RMS_LAUNCH(512, 8);
    else if (N <= 8192) ZK_RMS_LAUNCH(ZK_RMS_T8K, ZK_RMS_E8K);
    else if (N <= 16384) ZK_RMS_LAUNCH(1024, 16);
    else {
        rms_stat_kernel<<<grid, dim3(kRmsThreads), 0, 0>>>(A, rms, N, eps, dim);
        if (check_launch(name)) launch_apply<WT>(name, A, W, rms, C, M, N);
        return;
    }
#undef ZK_RMS_LAUNCH
    check_launch(name);
}

}  // namespace zk

extern "C" {

void rms_norm_32(const int64_t *A, const int32_t *W, const int64_t *rms, int64_t *C, int seqLen, int Dim)
{
    zk::launch_apply<int32_t>("rms_norm_32", A, W, rms, C, seqLen, Dim);
}

void rms_norm_64(const int64_t *A, const int64_t *W, const int64_t *rms, int64_t *C, int seqLen, int Dim)
{
    zk::launch_apply<int64_t>("rms_norm_64", A, W, rms, C, seqLen, Dim);
}

void rms_stat_int64(const int64_t *A, int64_t *rms, int M, int N, int64_t eps, int64_t dim)
{
    if (!zk::rms_args_ok("rms_stat_int64", A, nullptr, rms, nullptr, M, N) || !zk::stat_args_ok("rms_stat_int64", eps, dim))
        return;
    zk::rms_stat_kernel<<<dim3((unsigned)M), dim3(zk::kRmsThreads), 0, 0>>>(A, rms, N, eps, dim);
    zk::check_launch("rms_stat_int64");
}

void rms_norm_fused_32(const int64_t *A, const int32_t *W, int64_t *rms, int64_t *C, int M, int N, int64_t eps,
                       int64_t dim)
{
    zk::launch_fused<int32_t>("rms_norm_fused_32", A, W, rms, C, M, N, eps, dim);
}

void rms_norm_fused_64(const int64_t *A, const int64_t *W, int64_t *rms, int64_t *C, int M, int N, int64_t eps,
                       int64_t dim)
{
    zk::launch_fused<int64_t>("rms_norm_fused_64", A, W, rms, C, M, N, eps, dim);
}

}  // extern "C"
