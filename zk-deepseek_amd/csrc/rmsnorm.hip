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

// floor(x / d), d > 0.  32-bit divisors use schoolbook division on 32-bit digits; below 2^20 (every model shape:
// the row length) a digit step is a double-precision estimate and one correction.  This runs on one lane while the
// rest of the row's workgroup waits, so its length is the latency of a short launch.
__device__ U192 u192_div(U192 x, uint64_t d)
{
    U192 q;
    if (d < (1ull << 20)) {
        const uint32_t dig[6] = { (uint32_t)x.w0, (uint32_t)(x.w0 >> 32), (uint32_t)x.w1,
                                  (uint32_t)(x.w1 >> 32), (uint32_t)x.w2, (uint32_t)(x.w2 >> 32) };
        uint32_t qd[6];
        const double inv = 1.0 / (double)d;
        uint64_t rem = 0;
#pragma unroll
        for (int i = 5; i >= 0; i--) {
            // cur < 2^52 is exact as a double and cur / d < 2^32: the estimate is off by less than 2^-20, its floor by
            // at most one either way
            const uint64_t cur = (rem << 32) | dig[i];
            uint64_t qi = (uint64_t)((double)cur * inv);
            int64_t r = (int64_t)(cur - qi * d);
            if (r < 0) { qi--; r += (int64_t)d; }
            else if (r >= (int64_t)d) { qi++; r -= (int64_t)d; }
            qd[i] = (uint32_t)qi;
            rem = (uint64_t)r;
        }
        q.w0 = qd[0] | ((uint64_t)qd[1] << 32);
        q.w1 = qd[2] | ((uint64_t)qd[3] << 32);
        q.w2 = qd[4] | ((uint64_t)qd[5] << 32);
    } else if (d <= 0xFFFFFFFFull) {
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
// Written as a shift-and-subtract loop on the magnitudes: this is the rare last resort, and a compact loop keeps
// its register needs (which every kernel that contains it would inherit) next to nothing.
__device__ __forceinline__ int64_t rms_apply_slow(int64_t a, int64_t w, int64_t r)
{
    if (r == 0) return 0;
    const i128 prod = (i128)a * (i128)w;
    const bool pneg = prod < 0;
    const u128 up = pneg ? (u128)0 - (u128)prod : (u128)prod;
    const uint64_t ur = r < 0 ? 0 - (uint64_t)r : (uint64_t)r;
    uint64_t qh = 0, ql = 0, plo = (uint64_t)up, phi = (uint64_t)(up >> 64);
    uint64_t rem = 0;                 // stays below ur <= 2^63, so doubling it cannot overflow 64 bits
#pragma unroll 1
    for (int bit = 0; bit < 128; bit++) {
        rem = (rem << 1) | (phi >> 63);
        phi = (phi << 1) | (plo >> 63);
        plo <<= 1;
        qh = (qh << 1) | (ql >> 63);
        ql <<= 1;
        if (rem >= ur) { rem -= ur; ql |= 1; }
    }
    u128 uq = ((u128)qh << 64) | ql;
    // C++ semantics: the quotient truncates toward zero and the remainder takes the sign of the product
    u128 qq = (pneg != (r < 0)) ? (u128)0 - uq : uq;
    if (pneg && rem != 0) qq -= 1;
    return (int64_t)(uint64_t)qq;
}

// Three tiers, each exact where it answers.
//
// The quotient x = a*w/r is estimated in double precision from the operands themselves,
// xd = fl(fl(fl(a) * fl(w)) * fl(1 / fl(r))): six roundings of relative size 2^-53 at most, so |xd - x| <= |x| * 2^-50.
//
// Quick tier: n = floor(xd) is floor(x) whenever xd lies further than m = |xd| * 2^-49 (twice the bound and more)
// from both n and n + 1; a zero product is exact as it is.  This is all most elements ever run.
//
// Remainder tier, 0 < r < 2^62 and |x| < 2^49: the estimate is off by less than 2^49 * 2^-50 = 0.5, so rounded to
// nearest it lands within one of the floor; the remainder a*w - q*r, exact modulo 2^64, settles which.  The rounding
// and the conversion to an integer are one addition: for |x| < 2^51 the low bits of x + 1.5 * 2^52 hold round(x) as
// a fixed-point number.
//
// Anything else is divided the long way (rms_apply_slow).
template <typename WT>
__device__ __forceinline__ int64_t rms_apply_quick(int64_t a, WT w, double inv_r, bool fast_r, bool &certain)
{
    const double xd = (double)a * (double)w * inv_r;
    const double fl = floor(xd);
    const double frac = xd - fl;                     // exact
    const double m = fabs(xd) * 0x1p-49;             // >= 1 once |xd| >= 2^49: such elements are never certain
    certain = fast_r && ((frac > m && 1.0 - frac > m) || xd == 0.0);
    const double magic = 6755399441055744.0;
    return (int64_t)((uint64_t)__double_as_longlong(fl + magic) - (uint64_t)__double_as_longlong(magic));
}

template <typename WT>
__device__ __forceinline__ int64_t rms_apply_fast(int64_t a, WT w, int64_t r, double inv_r, bool fast_r, bool &ok)
{
    // straight-line code: estimate, remainder, one-step correction by selects; `ok` says whether the result stands
    const double xd = (double)a * (double)w * inv_r;
    const double magic = 6755399441055744.0;
    // (unsigned arithmetic throughout: a wild estimate must wrap, not overflow, on its way to being rejected)
    uint64_t q = (uint64_t)__double_as_longlong(xd + magic) - (uint64_t)__double_as_longlong(magic);
    const uint64_t plo = (uint64_t)a * (uint64_t)(int64_t)w;
    uint64_t rem = plo - q * (uint64_t)r;
    const bool neg = (int64_t)rem < 0, big = !neg && (int64_t)rem >= r;
    q += big ? 1ull : (neg ? ~0ull : 0ull);
    rem += neg ? (uint64_t)r : (big ? 0 - (uint64_t)r : 0ull);
    ok = fast_r && fabs(xd) < 562949953421312.0 && (int64_t)rem >= 0 && (int64_t)rem < r;
    return (int64_t)q;
}

template <typename WT>
__device__ __forceinline__ int64_t rms_apply_one(int64_t a, WT w, int64_t r, double inv_r, bool fast_r)
{
    bool ok;
    const int64_t q = rms_apply_fast(a, w, r, inv_r, fast_r, ok);
    if (__builtin_expect(!ok, 0)) return rms_apply_slow(a, (int64_t)w, r);
    return q;
}

// two consecutive weights in one load (the callers guarantee an even index and 16-byte aligned rows; the weight
// vector itself is only assumed to be aligned to its element size, so int64 weights stay two loads)
template <typename WT> struct WPair { WT x, y; };
template <typename WT>
__device__ __forceinline__ WPair<WT> load_w_pair(const WT *W, int i, bool w_vec)
{
    if (sizeof(WT) == 4 && w_vec) {
        const uint2 t = *reinterpret_cast<const uint2 *>(W + i);
        return { (WT)(int32_t)t.x, (WT)(int32_t)t.y };
    }
    return { W[i], W[i + 1] };
}

constexpr int kRmsThreads = 256;

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

typedef int v4i_r __attribute__((ext_vector_type(4)));

// Statistic only: one workgroup per row, any N.
__global__ __launch_bounds__(kRmsThreads) void rms_stat_kernel(const int64_t *__restrict__ A, int64_t *__restrict__ rms,
                                                               int N, int64_t eps, int64_t dim)
{
    __shared__ U192 red[kRmsThreads / 64];
    const int64_t *a = A + (long)blockIdx.x * N;
    SquareSum sq;
    if (N % 2 == 0 && ((uintptr_t)A & 15) == 0) {
        // two elements per load, four loads in flight per thread
        const int pairs = N / 2;
        int i = threadIdx.x;
        for (; i + 3 * kRmsThreads < pairs; i += 4 * kRmsThreads) {
            v4i_r t[4];
#pragma unroll
            for (int u = 0; u < 4; u++)
                t[u] = __builtin_nontemporal_load(reinterpret_cast<const v4i_r *>(a) + i + u * kRmsThreads);
#pragma unroll
            for (int u = 0; u < 4; u++) {
                sq.add((int64_t)(((uint64_t)(uint32_t)t[u][1] << 32) | (uint32_t)t[u][0]));
                sq.add((int64_t)(((uint64_t)(uint32_t)t[u][3] << 32) | (uint32_t)t[u][2]));
            }
        }
        for (; i < pairs; i += kRmsThreads) {
            const v4i_r t = __builtin_nontemporal_load(reinterpret_cast<const v4i_r *>(a) + i);
            sq.add((int64_t)(((uint64_t)(uint32_t)t[1] << 32) | (uint32_t)t[0]));
            sq.add((int64_t)(((uint64_t)(uint32_t)t[3] << 32) | (uint32_t)t[2]));
        }
    } else {
        for (int i = threadIdx.x; i < N; i += kRmsThreads) sq.add(a[i]);
    }
    U192 tot = block_sum_u192<kRmsThreads>(sq.total(), red);
    if (threadIdx.x == 0) rms[blockIdx.x] = rms_finalize(tot, eps, dim);
}

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
        WPair<WT> wp[kApplyEpt / 2];
        const bool w_vec = ((uintptr_t)W & 7) == 0;
        unsigned redo = 0;
#pragma unroll
        for (int j = 0; j < kApplyEpt / 2; j++) {
            const int i = base + (j * kRmsThreads + threadIdx.x) * 2;
            if (i < N) {
                t[j] = __builtin_nontemporal_load(reinterpret_cast<const v4i_r *>(a + i));
                wp[j] = load_w_pair(W, i, w_vec);
            }
        }
#pragma unroll
        for (int j = 0; j < kApplyEpt / 2; j++) {
            const int i = base + (j * kRmsThreads + threadIdx.x) * 2;
            if (i < N) {
                const int64_t v0 = (int64_t)(((uint64_t)(uint32_t)t[j][1] << 32) | (uint32_t)t[j][0]);
                const int64_t v1 = (int64_t)(((uint64_t)(uint32_t)t[j][3] << 32) | (uint32_t)t[j][2]);
                bool ok0, ok1;
                const int64_t c0 = rms_apply_quick(v0, wp[j].x, inv_r, fast_r, ok0);
                const int64_t c1 = rms_apply_quick(v1, wp[j].y, inv_r, fast_r, ok1);
                redo |= (ok0 ? 0u : 1u << (2 * j)) | (ok1 ? 0u : 2u << (2 * j));
                const v4i_r o = { (int)(uint32_t)c0, (int)(uint32_t)((uint64_t)c0 >> 32), (int)(uint32_t)c1,
                                  (int)(uint32_t)((uint64_t)c1 >> 32) };
                __builtin_nontemporal_store(o, reinterpret_cast<v4i_r *>(c + i));
            }
        }
        // rare: elements the quick tier could not settle go through the other two and are stored again
        if (__builtin_expect(redo != 0, 0)) {
#pragma unroll
            for (int j = 0; j < kApplyEpt / 2; j++) {
                const int i = base + (j * kRmsThreads + threadIdx.x) * 2;
                const int64_t v0 = (int64_t)(((uint64_t)(uint32_t)t[j][1] << 32) | (uint32_t)t[j][0]);
                const int64_t v1 = (int64_t)(((uint64_t)(uint32_t)t[j][3] << 32) | (uint32_t)t[j][2]);
                if (redo & (1u << (2 * j))) c[i] = rms_apply_one(v0, wp[j].x, r, inv_r, fast_r);
                if (redo & (2u << (2 * j))) c[i + 1] = rms_apply_one(v1, wp[j].y, r, inv_r, fast_r);
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
// WPE: waves per SIMD the register allocation must leave room for.  Rows of 4K-8K elements run three workgroups of
// eight waves per compute unit (WPE 6, 80 registers): measured, a third row in flight pays; a fourth (64 registers)
// spills again and does not.
// RES: the row that is normalised is A + Y * 2^k (wrapping int64 arithmetic, as the tensor ops of the reference's
// residual connection, inference/model.py:1465, 1472), and that sum is also stored to Xout (which may be A itself).
struct RmsResidual { const int64_t *Y; int64_t *Xout; int k; };

template <typename WT, int THREADS, int EPT, bool VEC, int WPE, bool RES>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(WPE))) void rms_fused_kernel(const int64_t *A, const WT *__restrict__ W,
                                                                int64_t *__restrict__ rms, int64_t *__restrict__ C,
                                                                int N, int64_t eps, int64_t dim, RmsResidual res)
{
    __shared__ U192 red[THREADS / 64];
    __shared__ int64_t rms_s;
    const long row = blockIdx.x;
    const int64_t *a = A + row * N;
    int64_t v[EPT];
    // The weights travel with the row: no load is left for after the barrier.  Where several rows share a compute unit
    // through a tight register budget (WPE > 1), int32 weights wait in LDS instead of registers (each thread reads
    // back only what it wrote itself): the registers they held were being spilled to scratch memory, and those
    // stores reached HBM (a tenth more bytes written than the output has).
    constexpr bool W_LDS = VEC && sizeof(WT) == 4 && WPE > 1;
    __shared__ WPair<WT> w_s[W_LDS ? (EPT / 2) * THREADS : 1];
    WPair<WT> wp[W_LDS ? 1 : EPT / 2];
    const bool w_vec = ((uintptr_t)W & 7) == 0;
    SquareSum sq;
    if (VEC) {
#pragma unroll
        for (int j = 0; j < EPT / 2; j++) {
            const int i = (j * THREADS + threadIdx.x) * 2;
            if (i < N) {
                const v4i_r t = __builtin_nontemporal_load(reinterpret_cast<const v4i_r *>(a + i));
                if (W_LDS) w_s[j * THREADS + threadIdx.x] = load_w_pair(W, i, w_vec);
                else wp[j] = load_w_pair(W, i, w_vec);
                v[2 * j] = (int64_t)(((uint64_t)(uint32_t)t[1] << 32) | (uint32_t)t[0]);
                v[2 * j + 1] = (int64_t)(((uint64_t)(uint32_t)t[3] << 32) | (uint32_t)t[2]);
                if (RES) {
                    const v4i_r u = __builtin_nontemporal_load(reinterpret_cast<const v4i_r *>(res.Y + row * N + i));
                    const uint64_t y0 = ((uint64_t)(uint32_t)u[1] << 32) | (uint32_t)u[0];
                    const uint64_t y1 = ((uint64_t)(uint32_t)u[3] << 32) | (uint32_t)u[2];
                    v[2 * j] = (int64_t)((uint64_t)v[2 * j] + (y0 << res.k));
                    v[2 * j + 1] = (int64_t)((uint64_t)v[2 * j + 1] + (y1 << res.k));
                    const v4i_r o = { (int)(uint32_t)v[2 * j], (int)(uint32_t)((uint64_t)v[2 * j] >> 32),
                                      (int)(uint32_t)v[2 * j + 1], (int)(uint32_t)((uint64_t)v[2 * j + 1] >> 32) };
                    __builtin_nontemporal_store(o, reinterpret_cast<v4i_r *>(res.Xout + row * N + i));
                }
                sq.add(v[2 * j]);
                sq.add(v[2 * j + 1]);
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < EPT; j++) {
            const int i = j * THREADS + threadIdx.x;
            if (i < N) {
                v[j] = a[i];
                if (RES) {
                    v[j] = (int64_t)((uint64_t)v[j] + ((uint64_t)res.Y[row * N + i] << res.k));
                    res.Xout[row * N + i] = v[j];
                }
                sq.add(v[j]);
            }
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
        unsigned redo = 0;
#pragma unroll
        for (int j = 0; j < EPT / 2; j++) {
            const int i = (j * THREADS + threadIdx.x) * 2;
            if (i < N) {
                bool ok0, ok1;
                const WPair<WT> w = W_LDS ? w_s[j * THREADS + threadIdx.x] : wp[W_LDS ? 0 : j];
                const int64_t c0 = rms_apply_quick(v[2 * j], w.x, inv_r, fast_r, ok0);
                const int64_t c1 = rms_apply_quick(v[2 * j + 1], w.y, inv_r, fast_r, ok1);
                redo |= (ok0 ? 0u : 1u << (2 * j)) | (ok1 ? 0u : 2u << (2 * j));
                const v4i_r t = { (int)(uint32_t)c0, (int)(uint32_t)((uint64_t)c0 >> 32), (int)(uint32_t)c1,
                                  (int)(uint32_t)((uint64_t)c1 >> 32) };
                __builtin_nontemporal_store(t, reinterpret_cast<v4i_r *>(C + row * N + i));
            }
        }
        // rare: elements the quick tier could not settle go through the other two and are stored again
        if (__builtin_expect(redo != 0, 0)) {
#pragma unroll
            for (int j = 0; j < EPT / 2; j++) {
                const int i = (j * THREADS + threadIdx.x) * 2;
                const WPair<WT> w = W_LDS ? w_s[j * THREADS + threadIdx.x] : wp[W_LDS ? 0 : j];
                if (redo & (1u << (2 * j))) C[row * N + i] = rms_apply_one(v[2 * j], w.x, r, inv_r, fast_r);
                if (redo & (2u << (2 * j))) C[row * N + i + 1] = rms_apply_one(v[2 * j + 1], w.y, r, inv_r, fast_r);
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

// Y * 2^k added to A, element by element (only for rows too long for the fused kernel)
__global__ __launch_bounds__(256) void residual_add_kernel(const int64_t *A, const int64_t *__restrict__ Y, int64_t *Xout, long n, int k)
{
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256)
        Xout[i] = (int64_t)((uint64_t)A[i] + ((uint64_t)Y[i] << k));
}

template <typename WT>
static void launch_fused(const char *name, const int64_t *A, const WT *W, int64_t *rms, int64_t *C, int M, int N,
                         int64_t eps, int64_t dim, const RmsResidual *res = nullptr)
{
    if (!rms_args_ok(name, A, W, rms, C, M, N) || !stat_args_ok(name, eps, dim)) return;
    if (!W) { set_error(kBadArgument, "%s: null pointer", name); return; }
    uintptr_t align = (uintptr_t)A | (uintptr_t)C;
    RmsResidual r = { nullptr, nullptr, 0 };
    if (res) {
        if (!res->Y || !res->Xout) { set_error(kBadArgument, "%s: null pointer", name); return; }
        if (res->k < 0 || res->k > 63) { set_error(kBadArgument, "%s: shift %d outside 0..63", name, res->k); return; }
        r = *res;
        align |= (uintptr_t)r.Y | (uintptr_t)r.Xout;
    }
    const bool vec = N % 2 == 0 && (align & 15) == 0;
    const dim3 grid((unsigned)M);
#define ZK_RMS_LAUNCH2(THREADS, EPT, WPE, VEC, RES) \
    rms_fused_kernel<WT, THREADS, EPT, VEC, WPE, RES><<<grid, dim3(THREADS), 0, 0>>>(A, W, rms, C, N, eps, dim, r)
#define ZK_RMS_LAUNCH(THREADS, EPT, WPE)                                                   \
    do {                                                                                   \
        if (res) { if (vec) ZK_RMS_LAUNCH2(THREADS, EPT, WPE, true, true); else ZK_RMS_LAUNCH2(THREADS, EPT, WPE, false, true); }    \
        else { if (vec) ZK_RMS_LAUNCH2(THREADS, EPT, WPE, true, false); else ZK_RMS_LAUNCH2(THREADS, EPT, WPE, false, false); }      \
    } while (0)
    if (N <= 512) ZK_RMS_LAUNCH(256, 2, 1);
    else if (N <= 2048) ZK_RMS_LAUNCH(256, 8, 1);
    else if (N <= 4096) ZK_RMS_LAUNCH(512, 8, 1);
    else if (N <= 8192) ZK_RMS_LAUNCH(512, 16, 6);
    else if (N <= 16384) ZK_RMS_LAUNCH(1024, 16, 1);
    else {
        const int64_t *src = A;
        if (res) {
            const long n = (long)M * N;
            residual_add_kernel<<<dim3((unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536)), dim3(256), 0, 0>>>(A, r.Y, r.Xout, n, r.k);
            if (!check_launch(name)) return;
            src = r.Xout;
        }
        rms_stat_kernel<<<grid, dim3(kRmsThreads), 0, 0>>>(src, rms, N, eps, dim);
        if (check_launch(name)) launch_apply<WT>(name, src, W, rms, C, M, N);
        return;
    }
#undef ZK_RMS_LAUNCH
#undef ZK_RMS_LAUNCH2
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

void rms_norm_residual_fused_32(const int64_t *X, const int64_t *Y, int k, const int32_t *W, int64_t *Xout, int64_t *rms,
                                int64_t *C, int M, int N, int64_t eps, int64_t dim)
{
    const zk::RmsResidual res = { Y, Xout, k };
    zk::launch_fused<int32_t>("rms_norm_residual_fused_32", X, W, rms, C, M, N, eps, dim, &res);
}

void rms_norm_residual_fused_64(const int64_t *X, const int64_t *Y, int k, const int64_t *W, int64_t *Xout, int64_t *rms,
                                int64_t *C, int M, int N, int64_t eps, int64_t dim)
{
    const zk::RmsResidual res = { Y, Xout, k };
    zk::launch_fused<int64_t>("rms_norm_residual_fused_64", X, W, rms, C, M, N, eps, dim, &res);
}

}  // extern "C"
