// Elementwise int64 fixed-point kernels: SiLU / sigmoid (Q23, Q25), the RoPE complex multiply and the
// three float -> fixed-point converters.  All are HBM-bound: 16-byte loads and stores, one pass.
#include "common.h"
#include "act_one.h"
#include "../../include/int64gemm.h"

namespace zk {

struct __attribute__((aligned(16))) i64x2 { int64_t x, y; };
typedef int v4i_e __attribute__((ext_vector_type(4)));

// Streaming 16-byte accesses (each byte is touched once): non-temporal, so they leave the caches alone.
__device__ __forceinline__ i64x2 ld_stream(const i64x2 *p)
{
    v4i_e t = __builtin_nontemporal_load(reinterpret_cast<const v4i_e *>(p));
    i64x2 r;
    r.x = (int64_t)(((uint64_t)(uint32_t)t[1] << 32) | (uint32_t)t[0]);
    r.y = (int64_t)(((uint64_t)(uint32_t)t[3] << 32) | (uint32_t)t[2]);
    return r;
}

__device__ __forceinline__ void st_stream(i64x2 *p, i64x2 v)
{
    v4i_e t = { (int)(uint32_t)v.x, (int)(uint32_t)((uint64_t)v.x >> 32), (int)(uint32_t)v.y, (int)(uint32_t)((uint64_t)v.y >> 32) };
    __builtin_nontemporal_store(t, reinterpret_cast<v4i_e *>(p));
}

// -------------------------------------------------------------------------------------------------
// SiLU / sigmoid.  sigma(x) = 1 / (1 + e^-x) with e^-x = 2^y, y = -x*log2(e) split into an integer part
// k (a shift) and a fraction looked up in a 256-entry table; the reciprocal is an exact integer divide.
// Follows inference/int64_gemm.cu:903-947, :969-1017 (Q23) and :775-819, :841-882 (Q25).
// -------------------------------------------------------------------------------------------------
constexpr int kActThreads = 256;
constexpr int kActUnroll = 4;

// GATED (SiLU only): C = (silu(R) * U) >> Q, the gate product of the FFNs (inference/model.py:1048, :1280), and
// the SiLU values themselves go to S when it is not null (the witness dump keeps them, model.py:1037-1042).
struct ActGate { const int64_t *U; int64_t *S; };

template <int Q>
__device__ __forceinline__ int64_t gate_mul(int64_t s, int64_t u) { return (int64_t)((uint64_t)s * (uint64_t)u) >> Q; }

template <int Q, bool SIGMOID, bool VEC, bool GATED>
__global__ __launch_bounds__(kActThreads) void act_kernel(const int64_t *__restrict__ R, int64_t *__restrict__ C,
                                                          const int64_t *__restrict__ lut_g, long n, ActGate gate)
{
    __shared__ int64_t lut[256];
    lut[threadIdx.x] = lut_g[threadIdx.x];
    __syncthreads();
    if (VEC) {
        long nvec = n >> 1;
        long base = (long)blockIdx.x * (kActThreads * kActUnroll) + threadIdx.x;
        i64x2 v[kActUnroll], u[GATED ? kActUnroll : 1];
#pragma unroll
        for (int j = 0; j < kActUnroll; j++) {
            long i = base + (long)j * kActThreads;
            if (i < nvec) {
                v[j] = ld_stream(reinterpret_cast<const i64x2 *>(R) + i);
                if (GATED) u[j] = ld_stream(reinterpret_cast<const i64x2 *>(gate.U) + i);
            }
        }
#pragma unroll
        for (int j = 0; j < kActUnroll; j++) {
            long i = base + (long)j * kActThreads;
            if (i < nvec) {
                i64x2 o;
                o.x = act_one<Q, SIGMOID>(v[j].x, lut);
                o.y = act_one<Q, SIGMOID>(v[j].y, lut);
                if (GATED) {
                    if (gate.S) st_stream(reinterpret_cast<i64x2 *>(gate.S) + i, o);
                    o.x = gate_mul<Q>(o.x, u[j].x);
                    o.y = gate_mul<Q>(o.y, u[j].y);
                }
                st_stream(reinterpret_cast<i64x2 *>(C) + i, o);
            }
        }
        if ((n & 1) && blockIdx.x == 0 && threadIdx.x == 0) {
            int64_t o = act_one<Q, SIGMOID>(R[n - 1], lut);
            if (GATED) { if (gate.S) gate.S[n - 1] = o; o = gate_mul<Q>(o, gate.U[n - 1]); }
            C[n - 1] = o;
        }
    } else {
        long base = (long)blockIdx.x * (kActThreads * kActUnroll) + threadIdx.x;
#pragma unroll
        for (int j = 0; j < kActUnroll; j++) {
            long i = base + (long)j * kActThreads;
            if (i < n) {
                int64_t o = act_one<Q, SIGMOID>(R[i], lut);
                if (GATED) { if (gate.S) gate.S[i] = o; o = gate_mul<Q>(o, gate.U[i]); }
                C[i] = o;
            }
        }
    }
}

// ---- large tensors: the reciprocal comes from a table ----------------------------------------------
// sigma depends on x only through the shift k and the table index of the fraction, so for the 2Q+2 shifts in
// [-(Q+1), Q] (every |x| below about 16.6 for Q23) the quotient 2^2Q / (2^Q + u) takes at most (2Q+2)*256
// values.  A pre-kernel computes them from the caller's table with the same integer arithmetic as act_one;
// the streaming kernel keeps them in LDS (48-52 KB) and does one 4-byte lookup per element instead of a
// divide.  Elements outside that range, or a table whose quotients do not fit 32 bits, take act_one.
//
// The quotients are kept from call to call (callers pass the same table every time) but never trusted: the
// pre-kernel leaves a copy of the table it worked from, every workgroup of the streaming kernel compares the
// caller's table with that copy while it loads it, and on a difference it divides per element like the small
// kernel and raises a flag in pinned host memory, which makes the next call build the quotients again.
template <int Q> struct QTab {
    static constexpr int kLo = -(Q + 1), kHi = Q, kRows = kHi - kLo + 1, kEntries = kRows * 256;
};

template <int Q>
__global__ __launch_bounds__(256) void act_qtab_kernel(const int64_t *__restrict__ lut, uint32_t *__restrict__ qtab,
                                                       int *__restrict__ ok, int64_t *__restrict__ lut_copy)
{
    constexpr int64_t ONE = (int64_t)1 << Q;
    const int k = QTab<Q>::kLo + (int)blockIdx.x;
    const int64_t t = lut[threadIdx.x];
    if (blockIdx.x == 0) lut_copy[threadIdx.x] = t;
    int64_t u;
    if (k < 0) u = t >> (-k);
    else u = (int64_t)((uint64_t)t << k);
    const int64_t den = (int64_t)((uint64_t)ONE + (uint64_t)u);
    const int64_t q = tdiv64((int64_t)1 << (2 * Q), den);
    qtab[blockIdx.x * 256 + threadIdx.x] = (uint32_t)q;
    // one flag per shift row (no cross-workgroup traffic): 1 when every quotient of the row fits 32 bits
    const int bad = __syncthreads_or(q < 0 || q > 0xFFFFFFFFll);
    if (threadIdx.x == 0) ok[blockIdx.x] = bad ? 0 : 1;
}

constexpr int kTabThreads = 512;

template <int Q, bool SIGMOID, bool GATED>
__global__ __launch_bounds__(kTabThreads) void act_table_kernel(const int64_t *__restrict__ R, int64_t *__restrict__ C,
                                                                const int64_t *__restrict__ lut_g,
                                                                const uint32_t *__restrict__ qtab_g,
                                                                const int *__restrict__ ok_g,
                                                                const int64_t *__restrict__ lut_copy_g, int *stale_host,
                                                                long n, ActGate gate)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char act_smem[];
    int64_t *lut = reinterpret_cast<int64_t *>(act_smem);
    uint32_t *qtab = reinterpret_cast<uint32_t *>(act_smem + 2048);
    constexpr int64_t LIM = (int64_t)64 << Q;
    constexpr int64_t ONE = (int64_t)1 << Q;
    int differs = 0;                     // the caller's table against the one the quotients were made from
    if (threadIdx.x < 256) {
        const int64_t t = lut_g[threadIdx.x];
        lut[threadIdx.x] = t;
        differs = t != lut_copy_g[threadIdx.x];
    }
    for (int i = threadIdx.x; i < QTab<Q>::kEntries / 4; i += kTabThreads)
        reinterpret_cast<v4i_e *>(qtab)[i] = reinterpret_cast<const v4i_e *>(qtab_g)[i];
    __shared__ int ok_s;
    if (threadIdx.x == 0) {
        int all = 1;
        for (int i = 0; i < QTab<Q>::kRows; i++) all &= ok_g[i];
        ok_s = all;
    }
    const int stale = __syncthreads_or(differs);
    const bool ok = ok_s != 0 && !stale;
    if (stale && stale_host && blockIdx.x == 0 && threadIdx.x == 0) *stale_host = 1;

    auto one = [&](int64_t r) -> int64_t {
        if (r >= LIM) return r;
        if (r <= -LIM) return 0;
        int64_t y;
        if (Q == 23) y = ((-r) * ActConst<Q>::kLog2e) >> Q;
        else y = -((r * ActConst<Q>::kLog2e) >> Q);
        const int k = (int)(y >> Q);
        if (!ok || k < QTab<Q>::kLo || k > QTab<Q>::kHi) return act_one<Q, SIGMOID>(r, lut);
        const int idx = (int)((y & (ONE - 1)) >> (Q - 8));
        const int64_t q = (int64_t)qtab[(k - QTab<Q>::kLo) * 256 + idx];
        if (SIGMOID) return q;
        return (r * q) >> Q;                 // |r| < 2^(Q+6), q <= 2^Q: exact in 64 bits
    };

    const long nvec = n >> 1;
    const long stride = (long)gridDim.x * (kTabThreads * kActUnroll);
    for (long base = (long)blockIdx.x * (kTabThreads * kActUnroll) + threadIdx.x; base < nvec; base += stride) {
        i64x2 v[kActUnroll], u[GATED ? kActUnroll : 1];
#pragma unroll
        for (int j = 0; j < kActUnroll; j++) {
            long i = base + (long)j * kTabThreads;
            if (i < nvec) {
                v[j] = ld_stream(reinterpret_cast<const i64x2 *>(R) + i);
                if (GATED) u[j] = ld_stream(reinterpret_cast<const i64x2 *>(gate.U) + i);
            }
        }
#pragma unroll
        for (int j = 0; j < kActUnroll; j++) {
            long i = base + (long)j * kTabThreads;
            if (i < nvec) {
                i64x2 o;
                o.x = one(v[j].x);
                o.y = one(v[j].y);
                if (GATED) {
                    if (gate.S) st_stream(reinterpret_cast<i64x2 *>(gate.S) + i, o);
                    o.x = gate_mul<Q>(o.x, u[j].x);
                    o.y = gate_mul<Q>(o.y, u[j].y);
                }
                st_stream(reinterpret_cast<i64x2 *>(C) + i, o);
            }
        }
    }
    if ((n & 1) && blockIdx.x == 0 && threadIdx.x == 0) {
        int64_t o = one(R[n - 1]);
        if (GATED) { if (gate.S) gate.S[n - 1] = o; o = gate_mul<Q>(o, gate.U[n - 1]); }
        C[n - 1] = o;
    }
}

// Per Q, kept for the process lifetime: (2Q+2)*256 quotients, the ok flags of their rows, the table they were made from.
constexpr size_t kQtabBytes = (size_t)QTab<25>::kEntries * 4;
constexpr size_t kQtabFlagBytes = (size_t)QTab<25>::kRows * 4;
constexpr size_t kQtabLutOffset = (kQtabBytes + kQtabFlagBytes + 15) & ~(size_t)15;
struct QtabCache { uint32_t *dev = nullptr; bool built = false; };
static QtabCache g_qtab_cache[2];       // Q23, Q25
static int *g_qtab_stale = nullptr;     // pinned host memory, one flag per Q: a streaming kernel met another table than the cached one
static bool g_qtab_stale_tried = false;

// Device memory held for the quotient tables, and its return (the tables are made again when next needed).
size_t act_workspace_bytes()
{
    size_t n = 0;
    for (const QtabCache &qc : g_qtab_cache) n += qc.dev ? kQtabLutOffset + 2048 : 0;
    return n;
}

void act_release_workspace()
{
    for (QtabCache &qc : g_qtab_cache) {
        if (qc.dev) (void)hipFree(qc.dev);
        qc.dev = nullptr;
        qc.built = false;
    }
}

template <int Q, bool SIGMOID, bool GATED = false>
static void launch_act(const char *name, const int64_t *R, int64_t *C, const int64_t *lut, int Bsz, int S, int Dim,
                       ActGate gate = ActGate{ nullptr, nullptr })
{
    if (Bsz < 0 || S < 0 || Dim < 0) { set_error(kBadArgument, "%s: negative dimension", name); return; }
    long n = (long)Bsz * S * Dim;
    if (n == 0) return;
    if (!R || !C || !lut || (GATED && !gate.U)) { set_error(kBadArgument, "%s: null pointer", name); return; }
    bool vec = (((uintptr_t)R | (uintptr_t)C | (uintptr_t)gate.U | (uintptr_t)gate.S) & 15) == 0;
    if (vec && n >= (1L << 20)) {
        QtabCache &qc = g_qtab_cache[Q == 23 ? 0 : 1];
        if (!qc.dev && hipMalloc(&qc.dev, kQtabLutOffset + 2048) != hipSuccess) {
            (void)hipGetLastError();
            qc.dev = nullptr;
        }
        if (!g_qtab_stale_tried) {
            g_qtab_stale_tried = true;
            if (hipHostMalloc(&g_qtab_stale, 2 * sizeof(int), hipHostMallocDefault) == hipSuccess) g_qtab_stale[0] = g_qtab_stale[1] = 0;
            else { (void)hipGetLastError(); g_qtab_stale = nullptr; }
        }
        if (qc.dev) {
            uint32_t *g_qtab = qc.dev;
            int *ok = reinterpret_cast<int *>(reinterpret_cast<unsigned char *>(g_qtab) + kQtabBytes);
            int64_t *lut_copy = reinterpret_cast<int64_t *>(reinterpret_cast<unsigned char *>(g_qtab) + kQtabLutOffset);
            // without the pinned flag nothing could report a changed table: the quotients are then made on every call
            int *stale = g_qtab_stale ? g_qtab_stale + (Q == 23 ? 0 : 1) : nullptr;
            if (!qc.built || !stale || *reinterpret_cast<volatile int *>(stale)) {
                if (stale) *reinterpret_cast<volatile int *>(stale) = 0;
                act_qtab_kernel<Q><<<dim3(QTab<Q>::kRows), dim3(256), 0, 0>>>(lut, g_qtab, ok, lut_copy);
                qc.built = true;
            }
            const size_t lds = 2048 + (size_t)QTab<Q>::kEntries * 4;
            static bool raised = false;
            if (!raised) {
                if (hipFuncSetAttribute((const void *)act_table_kernel<Q, SIGMOID, GATED>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)lds) != hipSuccess) {
                    set_error(kLaunchFailure, "%s: cannot raise the LDS limit", name);
                    return;
                }
                raised = true;
            }
            const long per_block = (long)kTabThreads * kActUnroll;
            long blocks = ((n >> 1) + per_block - 1) / per_block;
            // persistent workgroups, each loads the table once: two per CU; the gate product, with three or four streams
            // instead of two, runs fastest on 192 workgroups from some tens of millions of elements on (measured on one box
            // against 128 to 640: [1,8192,18432] 0.608 ms against 0.693 ms on 512, [1,2048,18432] 0.148 against 0.160,
            // [1,512,18432] 0.039 against 0.038)
            const long cap = (GATED && n >= (1L << 25)) ? 192 : 512;
            if (blocks > cap) blocks = cap;
            act_table_kernel<Q, SIGMOID, GATED><<<dim3((unsigned)blocks), dim3(kTabThreads), lds, 0>>>(R, C, lut, g_qtab, ok, lut_copy, stale, n, gate);
            check_launch(name);
            return;
        }
    }
    long per_block = (long)kActThreads * kActUnroll;
    long items = vec ? ((n >> 1) > 0 ? (n >> 1) : 1) : n;
    long blocks = (items + per_block - 1) / per_block;
    if (vec) act_kernel<Q, SIGMOID, true, GATED><<<dim3((unsigned)blocks), dim3(kActThreads), 0, 0>>>(R, C, lut, n, gate);
    else act_kernel<Q, SIGMOID, false, GATED><<<dim3((unsigned)blocks), dim3(kActThreads), 0, 0>>>(R, C, lut, n, gate);
    check_launch(name);
}

// -------------------------------------------------------------------------------------------------
// RoPE: (a0 + i a1) * (b0 + i b1) in Q42.  Each real product keeps bits [42,106) of the signed 128-bit
// product (inference/int64_gemm.cu:257-263); the table is broadcast over batch and heads (:245).
// -------------------------------------------------------------------------------------------------
__device__ __forceinline__ int64_t mul_q42(int64_t a, int64_t b)
{
    uint64_t lo = (uint64_t)a * (uint64_t)b;
    uint64_t hi = (uint64_t)__mul64hi((long long)a, (long long)b);
    return (int64_t)((hi << 22) | (lo >> 42));
}

__global__ __launch_bounds__(256) void rope_kernel(const i64x2 *__restrict__ A, const i64x2 *__restrict__ Bt,
                                                   i64x2 *__restrict__ C, long total, int seq, int heads, int headDim)
{
    long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    long i = idx;
    int d = (int)(i % headDim);
    i /= headDim;
    i /= heads;
    int s = (int)(i % seq);
    i64x2 a = A[idx];
    i64x2 b = Bt[(long)s * headDim + d];
    i64x2 o;
    o.x = (int64_t)((uint64_t)mul_q42(a.x, b.x) - (uint64_t)mul_q42(a.y, b.y));
    o.y = (int64_t)((uint64_t)mul_q42(a.x, b.y) + (uint64_t)mul_q42(a.y, b.x));
    C[idx] = o;
}

// -------------------------------------------------------------------------------------------------
// float bit patterns -> fixed point (inference/int64_gemm.cu:92-221).  value = (1.mantissa) * 2^(exp+rescale)
// truncated toward zero; shifts the reference leaves to the hardware are fixed as: left shift of 32 or more
// gives 0, right shift of 32 or more gives 0.
// -------------------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t scale_mantissa_u32(uint32_t r2, int ex2)
{
    // multiplying or dividing the (positive) mantissa by 1u << n is a shift
    if (ex2 >= 0) return ex2 >= 32 ? 0u : r2 << ex2;
    return -ex2 >= 31 ? 0u : r2 >> -ex2;
}

__device__ __forceinline__ int32_t bf16_one(uint32_t v0, int rescale, int wkv_b)
{
    const int ex0 = (int)((v0 >> 7) & 0xFF) - 127;
    const int r0 = (int)(v0 & 0x7F);
    if (ex0 == -127 && r0 == 0) return 0;
    if (wkv_b && ex0 >= -1) return 0x7FFFFFFF;                      // saturate |x| >= 0.5 (:151-154)
    uint32_t v = scale_mantissa_u32((uint32_t)(r0 + 128), ex0 + rescale);
    if (v0 & 0x8000) v = 0u - v;
    return (int32_t)v;
}

__device__ __forceinline__ int64_t f32_one(uint32_t v0, int rescale)
{
    const int ex0 = (int)((v0 >> 23) & 0xFF) - 127;
    const int r0 = (int)(v0 & 0x7FFFFF);
    if (ex0 == -127 && r0 == 0) return 0;
    const int ex2 = ex0 + rescale;
    const int64_t r2 = (int64_t)r0 + 8388608;
    int64_t v;
    // the reference multiplies by a 32-bit `1 << ex2` (:202): the factor wraps to INT_MIN at 31 and is 0 beyond
    // (shifts instead of the multiply and the divide: the mantissa is positive; at 31 the factor is -2^31)
    if (ex2 >= 0) v = ex2 >= 32 ? 0 : (ex2 == 31 ? (int64_t)(0 - ((uint64_t)r2 << 31)) : (int64_t)((uint64_t)r2 << ex2));
    else v = -ex2 >= 31 ? 0 : r2 >> -ex2;
    if (v0 & 0x80000000u) v = (int64_t)(0 - (uint64_t)v);
    return v;
}

typedef int v4i_e __attribute__((ext_vector_type(4)));

typedef int v2i_e __attribute__((ext_vector_type(2)));

// Four rounds per thread; in a round adjacent lanes handle adjacent groups of four bf16 values (8-byte load, 16-byte
// store), so loads and stores of a wavefront are both contiguous.  VEC: input 8-byte and output 16-byte aligned.
template <bool VEC>
__global__ __launch_bounds__(256) void bf16_to_int32_kernel(const uint16_t *__restrict__ in, int32_t *__restrict__ out,
                                                            long n, int rescale, int wkv_b)
{
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const long base = (((long)blockIdx.x * 4 + j) * 256 + threadIdx.x) * 4;
        if (base >= n) return;
        if (VEC && base + 4 <= n) {
            const v2i_e t = __builtin_nontemporal_load(reinterpret_cast<const v2i_e *>(in + base));
            v4i_e o;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const uint32_t w = (uint32_t)t[h];
                o[2 * h] = bf16_one(w & 0xFFFF, rescale, wkv_b);
                o[2 * h + 1] = bf16_one(w >> 16, rescale, wkv_b);
            }
            __builtin_nontemporal_store(o, reinterpret_cast<v4i_e *>(out + base));
        } else {
            for (long i = base; i < base + 4 && i < n; i++) out[i] = bf16_one(in[i], rescale, wkv_b);
        }
    }
}

// Same shape for fp32 -> int64: two values per lane and round (8-byte load, 16-byte store).
template <bool VEC>
__global__ __launch_bounds__(256) void f32_to_int64_kernel(const uint32_t *__restrict__ in, int64_t *__restrict__ out,
                                                           long n, int rescale)
{
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const long base = (((long)blockIdx.x * 4 + j) * 256 + threadIdx.x) * 2;
        if (base >= n) return;
        if (VEC && base + 2 <= n) {
            const v2i_e t = __builtin_nontemporal_load(reinterpret_cast<const v2i_e *>(in + base));
            const int64_t a = f32_one((uint32_t)t[0], rescale), b = f32_one((uint32_t)t[1], rescale);
            const v4i_e o = { (int)(uint32_t)a, (int)(uint32_t)((uint64_t)a >> 32), (int)(uint32_t)b, (int)(uint32_t)((uint64_t)b >> 32) };
            __builtin_nontemporal_store(o, reinterpret_cast<v4i_e *>(out + base));
        } else {
            for (long i = base; i < base + 2 && i < n; i++) out[i] = f32_one(in[i], rescale);
        }
    }
}

static void launch_bf16(const char *name, const uint16_t *input, int32_t *output, int rows, int cols, int rescale, int wkv_b)
{
    const long n = (long)rows * cols;
    if (rows < 0 || cols < 0) { set_error(kBadArgument, "%s: negative dimension", name); return; }
    if (n == 0) return;
    if (!input || !output) { set_error(kBadArgument, "%s: null pointer", name); return; }
    const long blocks = (n + 4095) / 4096;
    if (blocks > 0x7FFFFFFFL) { set_error(kUnsupportedSize, "%s: too many elements", name); return; }
    if (((uintptr_t)input & 7) == 0 && ((uintptr_t)output & 15) == 0)
        bf16_to_int32_kernel<true><<<dim3((unsigned)blocks), dim3(256), 0, 0>>>(input, output, n, rescale, wkv_b);
    else
        bf16_to_int32_kernel<false><<<dim3((unsigned)blocks), dim3(256), 0, 0>>>(input, output, n, rescale, wkv_b);
    check_launch(name);
}

}  // namespace zk

extern "C" {

void silu_q23(int64_t *R, int64_t *C, int64_t *lut, int Bsz, int S, int Dim)
{
    zk::launch_act<23, false>("silu_q23", R, C, lut, Bsz, S, Dim);
}
void sigmoid_q23(int64_t *R, int64_t *C, int64_t *lut, int Bsz, int S, int Dim)
{
    zk::launch_act<23, true>("sigmoid_q23", R, C, lut, Bsz, S, Dim);
}
void silu_q25(int64_t *R, int64_t *C, int64_t *lut, int Bsz, int S, int Dim)
{
    zk::launch_act<25, false>("silu_q25", R, C, lut, Bsz, S, Dim);
}
void sigmoid_q25(int64_t *R, int64_t *C, int64_t *lut, int Bsz, int S, int Dim)
{
    zk::launch_act<25, true>("sigmoid_q25", R, C, lut, Bsz, S, Dim);
}

void silu_mul_q23(const int64_t *R, const int64_t *U, int64_t *S, int64_t *C, const int64_t *lut, int Bsz, int Sq, int Dim)
{
    zk::launch_act<23, false, true>("silu_mul_q23", R, C, lut, Bsz, Sq, Dim, zk::ActGate{ U, S });
}

void complex_int64_mul(const int64_t *A, const int64_t *B, int64_t *C, int batchSize, int seqLen, int headCount,
                       int headDim)
{
    if (batchSize < 0 || seqLen < 0 || headCount < 0 || headDim < 0) {
        zk::set_error(zk::kBadArgument, "complex_int64_mul: negative dimension");
        return;
    }
    long total = (long)batchSize * seqLen * headCount * headDim;
    if (total == 0) return;
    if (!A || !B || !C) { zk::set_error(zk::kBadArgument, "complex_int64_mul: null pointer"); return; }
    if ((((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15) != 0) {
        zk::set_error(zk::kBadArgument, "complex_int64_mul: pointers must be 16-byte aligned");
        return;
    }
    long blocks = (total + 255) / 256;
    zk::rope_kernel<<<dim3((unsigned)blocks), dim3(256), 0, 0>>>(
        reinterpret_cast<const zk::i64x2 *>(A), reinterpret_cast<const zk::i64x2 *>(B),
        reinterpret_cast<zk::i64x2 *>(C), total, seqLen, headCount, headDim);
    zk::check_launch("complex_int64_mul");
}

void bf16_to_int32_2d(const uint16_t *input, int32_t *output, int rows, int cols, int rescale)
{
    zk::launch_bf16("bf16_to_int32_2d", input, output, rows, cols, rescale, 0);
}

void wkv_b_bf16_to_int32(const uint16_t *input, int32_t *output, int rows, int cols)
{
    zk::launch_bf16("wkv_b_bf16_to_int32", input, output, rows, cols, 25, 1);
}

void float32_to_int64_2d(const uint32_t *input, int64_t *output, int rows, int cols, int rescale)
{
    const char *name = "float32_to_int64_2d";
    const long n = (long)rows * cols;
    if (rows < 0 || cols < 0) { zk::set_error(zk::kBadArgument, "%s: negative dimension", name); return; }
    if (n == 0) return;
    if (!input || !output) { zk::set_error(zk::kBadArgument, "%s: null pointer", name); return; }
    const long blocks = (n + 2047) / 2048;
    if (blocks > 0x7FFFFFFFL) { zk::set_error(zk::kUnsupportedSize, "%s: too many elements", name); return; }
    if (((uintptr_t)input & 7) == 0 && ((uintptr_t)output & 15) == 0)
        zk::f32_to_int64_kernel<true><<<dim3((unsigned)blocks), dim3(256), 0, 0>>>(input, output, n, rescale);
    else
        zk::f32_to_int64_kernel<false><<<dim3((unsigned)blocks), dim3(256), 0, 0>>>(input, output, n, rescale);
    zk::check_launch(name);
}

}  // extern "C"
