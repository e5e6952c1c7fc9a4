// GEMM path (b): limb-decomposed i8 MFMA.
//
// Every int64 operand x is written in balanced base-256 digits, x = sum_j d_j * 256^j with d_j in [-128,127].
// The digits come from one 64-bit add and one xor: with bias_n = 0x80 in bytes 0..n-2,
//     d_j = byte_j(x + bias_n) - 128  (j < n-1),   d_{n-1} = signed byte_{n-1}(x + bias_n),
// which is exact whenever x + bias_n fits n signed bytes; n = 9 covers all of int64 (d_8 in {0,1}).
// The product sum then splits into digit-pair GEMMs that run on v_mfma_i32_32x32x32_i8,
//     sum_k a*b = sum_{i,j} 256^(i+j) * (sum_k da_i * db_j),
// all pairs with the same i+j share one int32 accumulator tile, and the epilogue recombines the
// NA+NB-1 diagonals with carries into the 128-bit sum before the shift.  Nothing is approximated.
//
// Operand tiles are converted on the fly: a thread loads 8 consecutive k of one row (64 bytes), splits them
// into digits with v_perm_b32 byte transposes and stores each digit plane to LDS already in MFMA fragment
// order (lane l of a fragment = row l%32, k-half l/32, 16 bytes), so the inner loop is ds_read_b128 + MFMA.
//
// The digit counts are speculated from a cached or sampled range; the workgroups of the first tile row /
// column track the exact min and max of everything they load, the launcher reads them back and reruns with
// wider digits in the rare case the guess was too small.  Results never depend on the guess.
#include "gemm.h"

#include <map>
#include <mutex>
#include <set>
#include <tuple>

namespace zk {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

struct MfmaParams {
    const int64_t *A;
    const void *B;
    int64_t *C, *R;
    long lda, sA, ldbn, ldbk, sB, ldc, sC;
    int M, N, K, shift;
    int64_t init;
    int tiles_m, tiles_n;
    unsigned long long *range;      // [minA, maxA, minB, maxB], order-preserving unsigned images of int64
    int verify_b_all_batches;       // B differs per batch: every batch's first tile row tracks its range
};

constexpr unsigned long long kSignFlip = 0x8000000000000000ull;

// ---- digit split -------------------------------------------------------------------------------
template <int N>
struct Limb {
    static constexpr uint64_t kBias = N >= 9 ? 0x8080808080808080ull
                                             : (N == 1 ? 0ull : (0x0080808080808080ull >> (8 * (8 - N))));
};

// 4x4 byte transpose: out[i] = bytes (y0.b_i, y1.b_i, y2.b_i, y3.b_i)
__device__ __forceinline__ void transpose4(uint32_t y0, uint32_t y1, uint32_t y2, uint32_t y3, uint32_t (&o)[4])
{
    uint32_t p01l = __builtin_amdgcn_perm(y1, y0, 0x05010400u);
    uint32_t p01h = __builtin_amdgcn_perm(y1, y0, 0x07030602u);
    uint32_t p23l = __builtin_amdgcn_perm(y3, y2, 0x05010400u);
    uint32_t p23h = __builtin_amdgcn_perm(y3, y2, 0x07030602u);
    o[0] = __builtin_amdgcn_perm(p23l, p01l, 0x05040100u);
    o[1] = __builtin_amdgcn_perm(p23l, p01l, 0x07060302u);
    o[2] = __builtin_amdgcn_perm(p23h, p01h, 0x05040100u);
    o[3] = __builtin_amdgcn_perm(p23h, p01h, 0x07060302u);
}

// x[0..7] (8 consecutive k of one row) -> out[i] = 8 bytes of digit i, k ascending.
template <int N>
__device__ __forceinline__ void limb_split8(const int64_t (&x)[8], uint2 (&out)[N])
{
    uint32_t lo[8], hi[8], e[8];
#pragma unroll
    for (int q = 0; q < 8; q++) {
        uint64_t u = (uint64_t)x[q] + Limb<N>::kBias;
        if (N >= 9) e[q] = (x[q] >= 0 && u < Limb<N>::kBias) ? 1u : 0u;
        u ^= Limb<N>::kBias;
        lo[q] = (uint32_t)u;
        hi[q] = (uint32_t)(u >> 32);
    }
    uint32_t t0[4], t1[4];
    transpose4(lo[0], lo[1], lo[2], lo[3], t0);
    transpose4(lo[4], lo[5], lo[6], lo[7], t1);
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (i < N) out[i] = make_uint2(t0[i], t1[i]);
    if (N > 4) {
        transpose4(hi[0], hi[1], hi[2], hi[3], t0);
        transpose4(hi[4], hi[5], hi[6], hi[7], t1);
#pragma unroll
        for (int i = 4; i < 8; i++)
            if (i < N) out[i] = make_uint2(t0[i - 4], t1[i - 4]);
    }
    if (N >= 9)
        out[N - 1] = make_uint2(e[0] | (e[1] << 8) | (e[2] << 16) | (e[3] << 24),
                                e[4] | (e[5] << 8) | (e[6] << 16) | (e[7] << 24));
}

// Smallest digit count whose range holds every value in [lo, hi].
static int limbs_needed(int64_t lo, int64_t hi)
{
    for (int n = 1; n <= 8; n++) {
        // x + bias_n in [-2^(8n-1), 2^(8n-1))
        i128 bias = n == 1 ? 0 : (i128)(0x0080808080808080ull >> (8 * (8 - n)));
        i128 half = (i128)1 << (8 * n - 1);
        if ((i128)lo + bias >= -half && (i128)hi + bias < half) return n;
    }
    return 9;
}

// ---- range tracking ------------------------------------------------------------------------------
struct MinMax { int64_t lo, hi; };

__device__ __forceinline__ void mm_update(MinMax &r, int64_t v)
{
    r.lo = v < r.lo ? v : r.lo;
    r.hi = v > r.hi ? v : r.hi;
}

__device__ __forceinline__ void mm_publish(MinMax r, unsigned long long *slot)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        int64_t ol = __shfl_xor(r.lo, off, kWave), oh = __shfl_xor(r.hi, off, kWave);
        r.lo = ol < r.lo ? ol : r.lo;
        r.hi = oh > r.hi ? oh : r.hi;
    }
    if ((threadIdx.x & 63) == 0) {
        atomicMin(slot, (unsigned long long)r.lo ^ kSignFlip);
        atomicMax(slot + 1, (unsigned long long)r.hi ^ kSignFlip);
    }
}

__global__ void range_reset_kernel(unsigned long long *range)
{
    if (threadIdx.x < 4) range[threadIdx.x] = (threadIdx.x & 1) ? 0ull : ~0ull;
}

// Strided sample of both operands for the first guess (at most `rows_s` rows x `cols_s` k each).
__global__ __launch_bounds__(256) void range_sample_kernel(MfmaParams p, int b32, int G, int which)
{
    MinMax r = { INT64_MAX, INT64_MIN };
    const long rows = which == 0 ? (long)p.M : (long)p.N;
    const long rstep = rows > 32 ? rows / 32 : 1;
    const long kstep = p.K > 256 ? p.K / 256 : 1;
    for (long ri = threadIdx.x >> 6; ri * rstep < rows && ri < 32; ri += 4) {
        long row = ri * rstep;
        for (long ki = threadIdx.x & 63; ki * kstep < p.K && ki < 256; ki += 64) {
            long k = ki * kstep;
            for (int g = 0; g < G; g += (G > 2 ? G / 2 : 1)) {
                int64_t v;
                if (which == 0) v = p.A[(long)g * p.sA + row * p.lda + k];
                else {
                    long off = (long)g * p.sB + row * p.ldbn + k * p.ldbk;
                    v = b32 ? (int64_t)reinterpret_cast<const int32_t *>(p.B)[off]
                            : reinterpret_cast<const int64_t *>(p.B)[off];
                }
                mm_update(r, v);
            }
        }
    }
    mm_publish(r, p.range + 2 * which);
}

// ---- the GEMM kernel -------------------------------------------------------------------------------
// WM x WN 32x32 MFMA tiles per wave, 2x2 waves per workgroup: workgroup tile (64*WM) x (64*WN), k-step 32.
template <int NA, int NB, int WM, int WN, bool B32, bool BKM>
__global__ __launch_bounds__(256, 1) void gemm_mfma_kernel(MfmaParams p)
{
    constexpr int BM = 64 * WM, BN = 64 * WN;
    constexpr int D = (NA + NB - 1) > 16 ? 16 : (NA + NB - 1);     // diagonal 16 has weight 2^128: dropped
    constexpr int A_BLOCKS = (BM / 32) * NA, B_BLOCKS = (BN / 32) * NB;
    constexpr int STAGE = (A_BLOCKS + B_BLOCKS) * 1024;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // workgroup -> tile.  Consecutive workgroup ids go to different XCDs (8 of them, each with its own L2), so
    // ids are regrouped to give each XCD a contiguous run of tiles; within a run the tile-row index moves
    // fastest, so the workgroups that share a B tile sit on the same L2.
    int bid = blockIdx.x;
    const int per_batch = p.tiles_m * p.tiles_n;
    const int total = per_batch * gridDim.y;
    int lin = blockIdx.y * per_batch + bid;
    if ((total & 7) == 0) lin = (lin & 7) * (total >> 3) + (lin >> 3);
    const int g = lin / per_batch;
    const int rem = lin - g * per_batch;
    const int tn = rem / p.tiles_m, tm = rem - tn * p.tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;

    const int64_t *Ag = p.A + (long)g * p.sA;
    const long boff = (long)g * p.sB;
    const bool verify_a = tn == 0;
    const bool verify_b = tm == 0 && (g == 0 || p.verify_b_all_batches);
    MinMax ra = { INT64_MAX, INT64_MIN }, rb = { INT64_MAX, INT64_MIN };

    v16i acc[WM][WN][D];
#pragma unroll
    for (int a = 0; a < WM; a++)
#pragma unroll
        for (int b = 0; b < WN; b++)
#pragma unroll
            for (int d = 0; d < D; d++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[a][b][d][r] = 0;

    // staging registers for the next k-step
    constexpr int A_IT = BM / 64, B_IT = BN / 64;
    int64_t sa[A_IT][8], sb[B_IT][8];

    // loader coordinates.  k-contiguous operands: 4 threads cover the 32 k of one row.  k-major B: 64 consecutive
    // threads cover 64 consecutive n of one k-octet.
    const int a_row = tid >> 2, a_oct = tid & 3;
    const int b_row = BKM ? (tid & 63) : (tid >> 2), b_oct = BKM ? (tid >> 6) : (tid & 3);
    const bool a_vec = (((uintptr_t)p.A | (uintptr_t)(p.lda * 8) | (uintptr_t)(p.sA * 8)) & 15) == 0;
    const bool b_vec = !BKM && (((uintptr_t)p.B | (uintptr_t)(p.ldbn * (B32 ? 4 : 8)) | (uintptr_t)(p.sB * (B32 ? 4 : 8))) & 15) == 0;

    auto fetch = [&](int k0) {
#pragma unroll
        for (int it = 0; it < A_IT; it++) {
            const int m = m0 + it * 64 + a_row, k = k0 + a_oct * 8;
            const int64_t *src = Ag + (long)m * p.lda + k;
            if (m < p.M && k + 8 <= p.K && a_vec) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const v4i t = reinterpret_cast<const v4i *>(src)[q];
                    sa[it][2 * q] = (int64_t)(((uint64_t)(uint32_t)t[1] << 32) | (uint32_t)t[0]);
                    sa[it][2 * q + 1] = (int64_t)(((uint64_t)(uint32_t)t[3] << 32) | (uint32_t)t[2]);
                }
            } else {
#pragma unroll
                for (int q = 0; q < 8; q++) sa[it][q] = (m < p.M && k + q < p.K) ? src[q] : 0;
            }
        }
#pragma unroll
        for (int it = 0; it < B_IT; it++) {
            const int n = n0 + it * 64 + b_row, k = k0 + b_oct * 8;
            if (BKM) {
#pragma unroll
                for (int q = 0; q < 8; q++) {
                    const long off = boff + n + (long)(k + q) * p.ldbk;
                    int64_t v = 0;
                    if (n < p.N && k + q < p.K)
                        v = B32 ? (int64_t)reinterpret_cast<const int32_t *>(p.B)[off]
                                : reinterpret_cast<const int64_t *>(p.B)[off];
                    sb[it][q] = v;
                }
            } else if (B32) {
                const int32_t *src = reinterpret_cast<const int32_t *>(p.B) + boff + (long)n * p.ldbn + k;
                if (n < p.N && k + 8 <= p.K && b_vec) {
#pragma unroll
                    for (int q = 0; q < 2; q++) {
                        const v4i t = reinterpret_cast<const v4i *>(src)[q];
#pragma unroll
                        for (int z = 0; z < 4; z++) sb[it][4 * q + z] = (int64_t)t[z];
                    }
                } else {
#pragma unroll
                    for (int q = 0; q < 8; q++) sb[it][q] = (n < p.N && k + q < p.K) ? (int64_t)src[q] : 0;
                }
            } else {
                const int64_t *src = reinterpret_cast<const int64_t *>(p.B) + boff + (long)n * p.ldbn + k;
                if (n < p.N && k + 8 <= p.K && b_vec) {
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const v4i t = reinterpret_cast<const v4i *>(src)[q];
                        sb[it][2 * q] = (int64_t)(((uint64_t)(uint32_t)t[1] << 32) | (uint32_t)t[0]);
                        sb[it][2 * q + 1] = (int64_t)(((uint64_t)(uint32_t)t[3] << 32) | (uint32_t)t[2]);
                    }
                } else {
#pragma unroll
                    for (int q = 0; q < 8; q++) sb[it][q] = (n < p.N && k + q < p.K) ? src[q] : 0;
                }
            }
        }
    };

    // digits of the staged rows -> LDS stage `buf`, fragment order
    auto stash = [&](int buf) {
        unsigned char *base = smem + buf * STAGE;
#pragma unroll
        for (int it = 0; it < A_IT; it++) {
            if (verify_a) {
#pragma unroll
                for (int q = 0; q < 8; q++) mm_update(ra, sa[it][q]);
            }
            uint2 dg[NA];
            limb_split8<NA>(sa[it], dg);
            const int row = it * 64 + a_row;
            const int slot = (row & 31) + 32 * (a_oct >> 1);
            unsigned char *dst = base + ((row >> 5) * NA) * 1024 + slot * 16 + (a_oct & 1) * 8;
#pragma unroll
            for (int i = 0; i < NA; i++) *reinterpret_cast<uint2 *>(dst + i * 1024) = dg[i];
        }
#pragma unroll
        for (int it = 0; it < B_IT; it++) {
            if (verify_b) {
#pragma unroll
                for (int q = 0; q < 8; q++) mm_update(rb, sb[it][q]);
            }
            uint2 dg[NB];
            limb_split8<NB>(sb[it], dg);
            const int row = it * 64 + b_row;
            const int slot = (row & 31) + 32 * (b_oct >> 1);
            unsigned char *dst = base + (A_BLOCKS + (row >> 5) * NB) * 1024 + slot * 16 + (b_oct & 1) * 8;
#pragma unroll
            for (int i = 0; i < NB; i++) *reinterpret_cast<uint2 *>(dst + i * 1024) = dg[i];
        }
    };

    auto compute = [&](int buf) {
        const unsigned char *base = smem + buf * STAGE;
        v4i fa[WM][NA], fb[WN][NB];
#pragma unroll
        for (int a = 0; a < WM; a++)
#pragma unroll
            for (int i = 0; i < NA; i++)
                fa[a][i] = *reinterpret_cast<const v4i *>(base + (((wm * WM + a) * NA + i) * 1024) + lane * 16);
#pragma unroll
        for (int b = 0; b < WN; b++)
#pragma unroll
            for (int j = 0; j < NB; j++)
                fb[b][j] = *reinterpret_cast<const v4i *>(base + ((A_BLOCKS + (wn * WN + b) * NB + j) * 1024) + lane * 16);
#pragma unroll
        for (int i = 0; i < NA; i++)
#pragma unroll
            for (int j = 0; j < NB; j++)
                if (i + j < D) {
#pragma unroll
                    for (int a = 0; a < WM; a++)
#pragma unroll
                        for (int b = 0; b < WN; b++)
                            acc[a][b][i + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[a][i], fb[b][j], acc[a][b][i + j], 0, 0, 0);
                }
    };

    const int ksteps = (p.K + 31) / 32;
    fetch(0);
    stash(0);
    __syncthreads();
    for (int ks = 0; ks < ksteps; ks++) {
        const int cur = ks & 1;
        if (ks + 1 < ksteps) fetch((ks + 1) * 32);
        compute(cur);
        if (ks + 1 < ksteps) stash(cur ^ 1);
        __syncthreads();
    }

    if (verify_a) mm_publish(ra, p.range);
    if (verify_b) mm_publish(rb, p.range + 2);

    // epilogue: diagonals -> 128-bit sum -> shift.  Accumulator register r of lane l holds
    // row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its 32x32 tile.
    const uint64_t rmask = p.shift ? ((1ull << p.shift) - 1) : 0;
#pragma unroll
    for (int a = 0; a < WM; a++) {
#pragma unroll
        for (int b = 0; b < WN; b++) {
            const int n = n0 + (wn * WN + b) * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + (wm * WM + a) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                uint64_t lo = (uint64_t)p.init, hi = (uint64_t)(p.init >> 63);
#pragma unroll
                for (int d = 0; d < D; d++) {
                    const int64_t v = (int64_t)acc[a][b][d][r];
                    uint64_t clo, chi;
                    if (d == 0) { clo = (uint64_t)v; chi = (uint64_t)(v >> 63); }
                    else if (d < 8) { clo = (uint64_t)v << (8 * d); chi = (uint64_t)(v >> (64 - 8 * d)); }
                    else if (d == 8) { clo = 0; chi = (uint64_t)v; }
                    else { clo = 0; chi = (uint64_t)v << (8 * (d - 8)); }
                    const uint64_t s = lo + clo;
                    hi += chi + (s < lo ? 1 : 0);
                    lo = s;
                }
                if (m < p.M && n < p.N) {
                    const long o = (long)g * p.sC + (long)m * p.ldc + n;
                    uint64_t q;
                    if (p.shift == 0) q = lo;
                    else q = (lo >> p.shift) | (hi << (64 - p.shift));
                    p.C[o] = (int64_t)q;
                    if (p.R) p.R[o] = (int64_t)(lo & rmask);
                }
            }
        }
    }
}

// ---- host side ---------------------------------------------------------------------------------------
typedef void (*MfmaKernel)(MfmaParams);

struct Instance {
    int na, nb, wm, wn;
    MfmaKernel fn[2][2];     // [b32][kmajor]
};

template <int NA, int NB, int WM, int WN>
static Instance make_instance()
{
    Instance s;
    s.na = NA; s.nb = NB; s.wm = WM; s.wn = WN;
    s.fn[0][0] = gemm_mfma_kernel<NA, NB, WM, WN, false, false>;
    s.fn[0][1] = gemm_mfma_kernel<NA, NB, WM, WN, false, true>;
    s.fn[1][0] = s.fn[1][1] = nullptr;
    if constexpr (NB <= 5) {          // int32 values never need more than five digits
        s.fn[1][0] = gemm_mfma_kernel<NA, NB, WM, WN, true, false>;
        s.fn[1][1] = gemm_mfma_kernel<NA, NB, WM, WN, true, true>;
    }
    return s;
}

// Digit-count combinations that are compiled.  A request is rounded up to the cheapest one that covers it.
static const Instance *instances(int *count)
{
    static const Instance table[] = {
        make_instance<3, 3, 2, 2>(), make_instance<4, 3, 2, 1>(), make_instance<4, 4, 2, 1>(),
        make_instance<5, 4, 2, 1>(), make_instance<5, 5, 2, 1>(), make_instance<6, 5, 2, 1>(),
        make_instance<3, 5, 2, 1>(), make_instance<6, 3, 2, 1>(),
        make_instance<9, 5, 1, 1>(), make_instance<5, 9, 1, 1>(), make_instance<9, 9, 1, 1>(),
    };
    *count = (int)(sizeof(table) / sizeof(table[0]));
    return table;
}

static const Instance *pick_instance(int na, int nb, bool b32)
{
    int count;
    const Instance *t = instances(&count);
    const Instance *best = nullptr;
    long best_cost = 0;
    for (int i = 0; i < count; i++) {
        if (t[i].na < na || t[i].nb < nb) continue;
        if (b32 && !t[i].fn[1][0]) continue;
        // MFMA work per output tile area, penalised a little for the smaller wave tiles
        long cost = (long)t[i].na * t[i].nb * 8 + (4 - t[i].wm * t[i].wn);
        if (!best || cost < best_cost) { best = &t[i]; best_cost = cost; }
    }
    return best;
}

struct RangeCache {
    std::mutex mu;
    std::map<std::tuple<const void *, long, long, int>, int> limbs;     // (ptr, rows, K, elem size) -> digits
    unsigned long long *dev = nullptr;
    int lookup(const void *ptr, long rows, long K, int esz)
    {
        auto it = limbs.find(std::make_tuple(ptr, rows, K, esz));
        return it == limbs.end() ? 0 : it->second;
    }
    void store(const void *ptr, long rows, long K, int esz, int n)
    {
        if (limbs.size() > 4096) limbs.clear();
        limbs[std::make_tuple(ptr, rows, K, esz)] = n;
    }
};

static RangeCache g_cache;

static bool read_range(unsigned long long *dev, int64_t (&out)[4])
{
    unsigned long long h[4];
    if (hipMemcpy(h, dev, sizeof(h), hipMemcpyDeviceToHost) != hipSuccess) return false;
    for (int i = 0; i < 4; i++) out[i] = (int64_t)(h[i] ^ kSignFlip);
    return true;
}

bool gemm_mfma_launch(const GemmDesc &d, int *limbs_a, int *limbs_b)
{
    if (d.a_rs != 1 || d.b_rs != 1) return false;                    // operand divisors: VALU path
    if (d.K <= 0 || d.M <= 0 || d.N <= 0 || d.G <= 0) return false;
    if (d.G > 65535) return false;
    const bool kmajor = d.ldbn == 1 && d.ldbk != 1;
    std::lock_guard<std::mutex> lock(g_cache.mu);
    if (!g_cache.dev) {
        if (hipMalloc(&g_cache.dev, 4 * sizeof(unsigned long long)) != hipSuccess) {
            set_error(kLaunchFailure, "gemm: cannot allocate the 32-byte range buffer");
            return false;
        }
    }

    MfmaParams p;
    p.A = d.A; p.B = d.B; p.C = d.C; p.R = d.R;
    p.lda = d.lda; p.sA = d.sA; p.ldbn = d.ldbn; p.ldbk = d.ldbk; p.sB = d.sB; p.ldc = d.ldc; p.sC = d.sC;
    p.M = d.M; p.N = d.N; p.K = d.K; p.shift = d.shift; p.init = d.init;
    p.range = g_cache.dev;
    p.verify_b_all_batches = d.sB != 0;

    const long rows_a = (long)d.G * d.M;
    int na = g_cache.lookup(d.A, rows_a, d.K, 8);
    int nb = g_cache.lookup(d.B, d.N, d.K, d.b32 ? 4 : 8);
    if (!na || !nb) {
        range_reset_kernel<<<1, 64, 0, 0>>>(p.range);
        range_sample_kernel<<<1, 256, 0, 0>>>(p, d.b32, d.G, 0);
        range_sample_kernel<<<1, 256, 0, 0>>>(p, d.b32, d.G, 1);
        int64_t r[4];
        if (!read_range(p.range, r)) { set_error(kLaunchFailure, "gemm: range readback failed"); return false; }
        if (!na) na = limbs_needed(r[0], r[1]);
        if (!nb) nb = limbs_needed(r[2], r[3]);
    }

    for (int attempt = 0; attempt < 3; attempt++) {
        const Instance *inst = pick_instance(na, nb, d.b32 != 0);
        if (!inst) return false;
        // int32 accumulators: at most min(NA,NB) digit pairs per diagonal, each product at most 2^14 in magnitude
        const long pairs = inst->na < inst->nb ? inst->na : inst->nb;
        const long kpad = ((long)d.K + 31) / 32 * 32;
        if (pairs * kpad * 16384 > 0x7FFFFFFFL) return false;
        MfmaKernel fn = inst->fn[d.b32 ? 1 : 0][kmajor ? 1 : 0];
        const int BM = 64 * inst->wm, BN = 64 * inst->wn;
        p.tiles_m = (d.M + BM - 1) / BM;
        p.tiles_n = (d.N + BN - 1) / BN;
        const long per_batch = (long)p.tiles_m * p.tiles_n;
        if (per_batch > 0x7FFFFFFFL) return false;
        const size_t lds = 2 * (size_t)((BM / 32) * inst->na + (BN / 32) * inst->nb) * 1024;
        static std::set<const void *> lds_raised;
        if (lds > 64 * 1024 && !lds_raised.count((const void *)fn)) {
            if (hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
                set_error(kLaunchFailure, "gemm: cannot raise the LDS limit to %zu bytes", lds);
                return false;
            }
            lds_raised.insert((const void *)fn);
        }
        range_reset_kernel<<<1, 64, 0, 0>>>(p.range);
        fn<<<dim3((unsigned)per_batch, (unsigned)d.G), dim3(256), lds, 0>>>(p);
        if (hipGetLastError() != hipSuccess) { set_error(kLaunchFailure, "gemm: MFMA kernel launch failed"); return false; }
        int64_t r[4];
        if (!read_range(p.range, r)) { set_error(kLaunchFailure, "gemm: range readback failed"); return false; }
        const int need_a = limbs_needed(r[0], r[1]), need_b = limbs_needed(r[2], r[3]);
        g_cache.store(d.A, rows_a, d.K, 8, need_a);
        g_cache.store(d.B, d.N, d.K, d.b32 ? 4 : 8, need_b);
        *limbs_a = inst->na;
        *limbs_b = inst->nb;
        if (need_a <= inst->na && need_b <= inst->nb) return true;
        na = need_a;
        nb = need_b;
    }
    set_error(kLaunchFailure, "gemm: digit count did not settle");
    return false;
}

}  // namespace zk
