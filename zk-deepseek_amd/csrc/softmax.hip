// Fixed-point row softmax over the last dimension of [Bsz,S,H,T] int64 (Q19 truncating, Q21 rounding).
//
// Rows of up to 2048 elements are handled one row per wavefront: the row is read once with 16-byte loads
// into registers, the maximum and the weight sum are 64-lane butterfly reductions, and the per-row divide
// is a reciprocal multiply made exact by a remainder test.  HBM traffic is the algorithmic 16 bytes per
// element (24 when the reference's write-back of the weights into the input is switched on).
// Longer rows use one workgroup per row and three passes.
//
// Arithmetic follows inference/int64_gemm.cu:684-746 (Q19) and :605-659 (Q21).
#include "common.h"
#include "../../include/int64gemm.h"

namespace zk {

static bool g_softmax_clobber = false;

struct __attribute__((aligned(16))) i64x2s { int64_t x, y; };
typedef int v4i_s __attribute__((ext_vector_type(4)));

// Streaming 16-byte accesses: every byte is touched exactly once, so the loads and stores are marked
// non-temporal and do not displace anything from the caches.
__device__ __forceinline__ i64x2s ld_stream(const i64x2s *p)
{
    v4i_s t = __builtin_nontemporal_load(reinterpret_cast<const v4i_s *>(p));
    i64x2s r;
    r.x = (int64_t)(((uint64_t)(uint32_t)t[1] << 32) | (uint32_t)t[0]);
    r.y = (int64_t)(((uint64_t)(uint32_t)t[3] << 32) | (uint32_t)t[2]);
    return r;
}

__device__ __forceinline__ void st_stream(i64x2s *p, i64x2s v)
{
    v4i_s t = { (int)(uint32_t)v.x, (int)(uint32_t)((uint64_t)v.x >> 32), (int)(uint32_t)v.y, (int)(uint32_t)((uint64_t)v.y >> 32) };
    __builtin_nontemporal_store(t, reinterpret_cast<v4i_s *>(p));
}

template <int Q>
__device__ __forceinline__ int64_t smx_weight(int64_t x, int64_t rmax, const int64_t *lut)
{
    if (Q == 19) {
        uint64_t d = (uint64_t)rmax - (uint64_t)x;                 // >= 0 by construction
        if (d > ((uint64_t)64 << 19)) return 0;
        uint64_t y = (d * 756388ull) >> 19;                        // d <= 2^25: the product is below 2^45
        uint64_t k = y >> 19;
        uint64_t f = y & 0x7FFFF;
        int64_t t = lut[f >> 11];
        return k >= 64 ? 0 : (t >> (int)k);
    } else {
        int64_t d = (int64_t)((uint64_t)x - (uint64_t)rmax);       // <= 0 unless the subtraction wrapped
        if (d < -((int64_t)64 << 21)) return 0;
        int64_t y = (int64_t)((uint64_t)d * 3025551ull + (1ull << 20)) >> 21;
        int64_t ny = (int64_t)(0 - (uint64_t)y);
        int64_t k = ny >> 21;
        int64_t f = ny & 0x1FFFFF;
        int64_t t = lut[f >> 13];
        if (k >= 64) return 0;
        return k < 0 ? (t >> 63) : (t >> (int)k);
    }
}

// Per-row divide.  fast: 2^12 <= s < 2^52 (true for every row whose maximum has weight LUT[0] = 2^Q).
template <int Q>
__device__ __forceinline__ int64_t smx_norm(int64_t w, int64_t s, double inv, bool fast)
{
    int64_t num = (int64_t)((uint64_t)w << Q);
    if (Q == 21) num = (int64_t)((uint64_t)num + (uint64_t)(s / 2));
    if (fast && w >= 0 && w < ((int64_t)1 << 30)) return (int64_t)udiv_by_inv((uint64_t)num, (uint64_t)s, inv);
    return s ? tdiv64(num, s) : 0;
}

constexpr int kSmxThreads = 256;

// Optional score preparation fused into the row load (inference/model.py:896-906 does it with three tensor ops):
//   x = floor((s1 + s2) * mul / div) + mask[s][t]
// s2, mask and scores (a copy of x for the witness dump, model.py:911-918) may be null.
struct SmxPre {
    const int64_t *s2;
    const int64_t *mask;      // [S, T], added to every batch and head
    int64_t *scores;
    int64_t mul, div;
    double inv_div;
    int S, H;
};

// floor(x / d) for 0 < d < 2^31 and any x: double estimate (exact to within one for |x| < 2^62, within a few
// otherwise) settled by the remainder
__device__ __forceinline__ int64_t floordiv_small(int64_t x, int64_t d, double inv_d)
{
    int64_t q = (int64_t)floor((double)x * inv_d);
    int64_t rem = (int64_t)((uint64_t)x - (uint64_t)q * (uint64_t)d);
    while (rem < 0) { q--; rem += d; }
    while (rem >= d) { q++; rem -= d; }
    return q;
}

__device__ __forceinline__ int64_t smx_prepare_value(int64_t v, int64_t s2, int64_t m, const SmxPre &pre)
{
    v = (int64_t)((uint64_t)v + (uint64_t)s2);
    v = (int64_t)((uint64_t)v * (uint64_t)pre.mul);
    if (pre.div != 1) v = floordiv_small(v, pre.div, pre.inv_div);
    return (int64_t)((uint64_t)v + (uint64_t)m);
}

template <bool PRE>
__device__ __forceinline__ int64_t smx_prepare(int64_t v, const SmxPre &pre, long row, int idx, int T)
{
    if (!PRE) return v;
    const long e = row * T + idx;
    v = smx_prepare_value(v, pre.s2 ? pre.s2[e] : 0, pre.mask ? pre.mask[(long)((row / pre.H) % pre.S) * T + idx] : 0, pre);
    if (pre.scores) pre.scores[e] = v;
    return v;
}

// two adjacent elements at once, every access 16 bytes wide (the caller has checked the alignment)
template <bool PRE>
__device__ __forceinline__ i64x2s smx_prepare_pair(i64x2s p, const SmxPre &pre, long row, int idx, int T)
{
    if (!PRE) return p;
    const long e = row * T + idx;
    i64x2s b = { 0, 0 }, m = { 0, 0 };
    if (pre.s2) b = ld_stream(reinterpret_cast<const i64x2s *>(pre.s2 + e));
    if (pre.mask) m = *reinterpret_cast<const i64x2s *>(pre.mask + (long)((row / pre.H) % pre.S) * T + idx);
    p.x = smx_prepare_value(p.x, b.x, m.x, pre);
    p.y = smx_prepare_value(p.y, b.y, m.y, pre);
    if (pre.scores) st_stream(reinterpret_cast<i64x2s *>(pre.scores + e), p);
    return p;
}

// One row per wavefront; EPL = elements per lane (even).  VEC: T is even and the pointers are 16-byte aligned.
template <int Q, int EPL, bool VEC, bool PRE>
__global__ __launch_bounds__(kSmxThreads) void softmax_wave_kernel(int64_t *__restrict__ R, int64_t *__restrict__ C,
                                                                   const int64_t *__restrict__ lut_g, long rows, int T,
                                                                   int clobber, SmxPre pre)
{
    __shared__ int64_t lut[256];
    lut[threadIdx.x] = lut_g[threadIdx.x];
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * (kSmxThreads / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    int64_t *x = R + row * T;
    int64_t *c = C + row * T;

    int64_t v[EPL];
    int64_t rmax = INT64_MIN;
#pragma unroll
    for (int j = 0; j < EPL / 2; j++) {
        int idx = (j * 64 + lane) * 2;
        if (VEC) {
            if (idx < T) {
                i64x2s p = ld_stream(reinterpret_cast<const i64x2s *>(x + idx));
                p = smx_prepare_pair<PRE>(p, pre, row, idx, T);
                v[2 * j] = p.x;
                v[2 * j + 1] = p.y;
                rmax = p.x > rmax ? p.x : rmax;
                rmax = p.y > rmax ? p.y : rmax;
            }
        } else {
            if (idx < T) { v[2 * j] = smx_prepare<PRE>(x[idx], pre, row, idx, T); rmax = v[2 * j] > rmax ? v[2 * j] : rmax; }
            if (idx + 1 < T) { v[2 * j + 1] = smx_prepare<PRE>(x[idx + 1], pre, row, idx + 1, T); rmax = v[2 * j + 1] > rmax ? v[2 * j + 1] : rmax; }
        }
    }
    rmax = wave_max_i64(rmax);

    uint64_t sum = 0;
#pragma unroll
    for (int j = 0; j < EPL; j++) {
        int idx = ((j >> 1) * 64 + lane) * 2 + (j & 1);
        if (idx < T) {
            v[j] = smx_weight<Q>(v[j], rmax, lut);
            sum += (uint64_t)v[j];
        }
    }
    const int64_t s = (int64_t)wave_sum_u64(sum);
    const bool fast = s >= ((int64_t)1 << 12) && s < ((int64_t)1 << 52);
    const double inv = fast ? 1.0 / (double)s : 0.0;

#pragma unroll
    for (int j = 0; j < EPL / 2; j++) {
        int idx = (j * 64 + lane) * 2;
        if (VEC) {
            if (idx < T) {
                i64x2s w, o;
                w.x = v[2 * j];
                w.y = v[2 * j + 1];
                o.x = smx_norm<Q>(w.x, s, inv, fast);
                o.y = smx_norm<Q>(w.y, s, inv, fast);
                st_stream(reinterpret_cast<i64x2s *>(c + idx), o);
                if (clobber) st_stream(reinterpret_cast<i64x2s *>(x + idx), w);
            }
        } else {
            if (idx < T) {
                c[idx] = smx_norm<Q>(v[2 * j], s, inv, fast);
                if (clobber) x[idx] = v[2 * j];
            }
            if (idx + 1 < T) {
                c[idx + 1] = smx_norm<Q>(v[2 * j + 1], s, inv, fast);
                if (clobber) x[idx + 1] = v[2 * j + 1];
            }
        }
    }
}

// One row per workgroup, any T: pass 1 maximum, pass 2 weights (staged in C) and their sum, pass 3 divide.
// Each thread re-reads only what it wrote itself, so the staging needs no fence.
template <int Q>
__global__ __launch_bounds__(kSmxThreads) void softmax_block_kernel(int64_t *__restrict__ R, int64_t *__restrict__ C,
                                                                    const int64_t *__restrict__ lut_g, int T, int clobber)
{
    __shared__ int64_t lut[256];
    __shared__ int64_t red[kSmxThreads / 64];
    lut[threadIdx.x] = lut_g[threadIdx.x];
    const long row = blockIdx.x;
    int64_t *x = R + row * T;
    int64_t *c = C + row * T;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

    int64_t rmax = INT64_MIN;
    for (int i = threadIdx.x; i < T; i += kSmxThreads) { int64_t a = x[i]; rmax = a > rmax ? a : rmax; }
    rmax = wave_max_i64(rmax);
    if (lane == 0) red[wave] = rmax;
    __syncthreads();
    rmax = red[0];
#pragma unroll
    for (int w = 1; w < kSmxThreads / 64; w++) rmax = red[w] > rmax ? red[w] : rmax;
    __syncthreads();

    uint64_t sum = 0;
    for (int i = threadIdx.x; i < T; i += kSmxThreads) {
        int64_t w = smx_weight<Q>(x[i], rmax, lut);
        c[i] = w;
        if (clobber) x[i] = w;
        sum += (uint64_t)w;
    }
    sum = wave_sum_u64(sum);
    if (lane == 0) red[wave] = (int64_t)sum;
    __syncthreads();
    uint64_t tot = 0;
#pragma unroll
    for (int w = 0; w < kSmxThreads / 64; w++) tot += (uint64_t)red[w];
    const int64_t s = (int64_t)tot;
    const bool fast = s >= ((int64_t)1 << 12) && s < ((int64_t)1 << 52);
    const double inv = fast ? 1.0 / (double)s : 0.0;
    for (int i = threadIdx.x; i < T; i += kSmxThreads) c[i] = smx_norm<Q>(c[i], s, inv, fast);
}

template <int Q, int EPL>
static void launch_wave(int64_t *R, int64_t *C, const int64_t *lut, long rows, int T, bool vec, int clobber, const SmxPre *pre)
{
    long blocks = (rows + (kSmxThreads / 64) - 1) / (kSmxThreads / 64);
    const dim3 grid((unsigned)blocks), block(kSmxThreads);
    SmxPre none = {};
    if (pre) {
        if (vec) softmax_wave_kernel<Q, EPL, true, true><<<grid, block, 0, 0>>>(R, C, lut, rows, T, clobber, *pre);
        else softmax_wave_kernel<Q, EPL, false, true><<<grid, block, 0, 0>>>(R, C, lut, rows, T, clobber, *pre);
    } else {
        if (vec) softmax_wave_kernel<Q, EPL, true, false><<<grid, block, 0, 0>>>(R, C, lut, rows, T, clobber, none);
        else softmax_wave_kernel<Q, EPL, false, false><<<grid, block, 0, 0>>>(R, C, lut, rows, T, clobber, none);
    }
}

// the score preparation as a pass of its own, for rows too long for the one-row-per-wavefront kernel
__global__ __launch_bounds__(256) void smx_prepare_kernel(const int64_t *__restrict__ s1, int64_t *__restrict__ out, long rows, int T, SmxPre pre)
{
    const long e = (long)blockIdx.x * 256 + threadIdx.x;
    if (e >= rows * T) return;
    SmxPre q = pre;
    q.scores = nullptr;
    out[e] = smx_prepare<true>(s1[e], q, e / T, (int)(e % T), T);
}

template <int Q>
static void launch_softmax(const char *name, int64_t *R, int64_t *C, const int64_t *lut, int Bsz, int S, int H, int T,
                           const SmxPre *pre = nullptr)
{
    if (Bsz < 0 || S < 0 || H < 0 || T < 0) { set_error(kBadArgument, "%s: negative dimension", name); return; }
    long rows = (long)Bsz * S * H;
    if (rows == 0 || T == 0) return;
    if (!R || !C || !lut) { set_error(kBadArgument, "%s: null pointer", name); return; }
    if (rows > 0x7FFFFFFFL) { set_error(kUnsupportedSize, "%s: more than 2^31-1 rows", name); return; }
    int clobber = g_softmax_clobber && !pre ? 1 : 0;
    bool vec = (T % 2 == 0) && ((((uintptr_t)R | (uintptr_t)C) & 15) == 0);
    if (pre && ((((uintptr_t)pre->s2 | (uintptr_t)pre->mask | (uintptr_t)pre->scores) & 15) != 0)) vec = false;
    if (T <= 128) launch_wave<Q, 2>(R, C, lut, rows, T, vec, clobber, pre);
    else if (T <= 256) launch_wave<Q, 4>(R, C, lut, rows, T, vec, clobber, pre);
    else if (T <= 512) launch_wave<Q, 8>(R, C, lut, rows, T, vec, clobber, pre);
    else if (T <= 1024) launch_wave<Q, 16>(R, C, lut, rows, T, vec, clobber, pre);
    else if (T <= 2048) launch_wave<Q, 32>(R, C, lut, rows, T, vec, clobber, pre);
    else {
        if (pre) {
            // long rows: prepared scores go to the scores buffer if there is one, else through C (the block kernel
            // reads all of a row before it writes any of it only when input and output differ, so C cannot serve as both)
            if (!pre->scores) { set_error(kBadArgument, "%s: rows longer than 2048 need a scores buffer", name); return; }
            const long n = rows * T;
            smx_prepare_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, 0>>>(R, pre->scores, rows, T, *pre);
            R = pre->scores;
        }
        softmax_block_kernel<Q><<<dim3((unsigned)rows), dim3(kSmxThreads), 0, 0>>>(R, C, lut, T, clobber);
    }
    check_launch(name);
}

}  // namespace zk

extern "C" {

void softmax_q19(int64_t *R, int64_t *C, int64_t *lut, int Bsz, int S, int H, int T)
{
    zk::launch_softmax<19>("softmax_q19", R, C, lut, Bsz, S, H, T);
}

void softmax_q21(int64_t *R, int64_t *C, int64_t *lut, int Bsz, int S, int H, int T)
{
    zk::launch_softmax<21>("softmax_q21", R, C, lut, Bsz, S, H, T);
}

void zk_softmax_clobber_input(int on) { zk::g_softmax_clobber = on != 0; }

void softmax_q19_scores(const int64_t *s1, const int64_t *s2, const int64_t *mask, int64_t *scores, int64_t *C,
                        const int64_t *lut, int Bsz, int S, int H, int T, int64_t mul, int64_t div)
{
    const char *name = "softmax_q19_scores";
    if (div <= 0 || div >= ((int64_t)1 << 31)) { zk::set_error(zk::kBadArgument, "%s: div must be in [1, 2^31)", name); return; }
    zk::SmxPre pre;
    pre.s2 = s2; pre.mask = mask; pre.scores = scores; pre.mul = mul; pre.div = div; pre.inv_div = 1.0 / (double)div;
    pre.S = S > 0 ? S : 1; pre.H = H > 0 ? H : 1;
    zk::launch_softmax<19>(name, const_cast<int64_t *>(s1), C, lut, Bsz, S, H, T, &pre);
}

}  // extern "C"
