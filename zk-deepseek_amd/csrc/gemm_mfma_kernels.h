// Device side of the limb-decomposed i8 MFMA GEMM (see gemm_mfma.hip for the scheme): digit split, loaders, the GEMM
// kernel, the split-K finish, the range kernels, and the table type that pairs a digit-count combination with its
// kernels.  The combinations are instantiated in several translation units (gemm_mfma_inst_*.hip) so that they
// compile side by side.
#pragma once
#include "gemm.h"
#include "../../include/int64gemm.h"

#include <type_traits>
#include <vector>

// Tuning knobs: MFMA depths (32 k each) per pipeline step by diagonal count, and how many vector-ALU
// instructions of the digit split are scheduled behind each MFMA of a step's last depth.  (A 32x32x32 MFMA holds the
// matrix pipe for 32 cycles, a vector instruction its own for 4; with two wavefronts on a SIMD up to four or five
// vector instructions per MFMA run in its shade, eight cost a quarter more time per MFMA: measured with a probe, and
// on the 512 x 7168 x 18432 product 0.631-0.638 ms with 5 against 0.642-0.643 with 8.)
#ifndef ZK_VALU_PER_MFMA
#define ZK_VALU_PER_MFMA 5
#endif
#ifndef ZK_KK
#define ZK_KK(DD) 1
#endif

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
    unsigned long long *range;      // [minA, maxA, minB, maxB], order-preserving unsigned images of int64; [4] verdict
    unsigned long long *wg_range;   // one such quadruple per workgroup of the GEMM kernel
    int verify_b_all_batches;       // B differs per batch: every batch's first tile row tracks its range
    const unsigned char *a_planes;  // pre-split digits of A (planes variants only)
    int a_msub, a_ksteps;           // 32-row groups and 32-k steps the planes were written for
    int b_nsub, b_ksteps;           // BPL kernels: B (or every group's B) is digit planes of that geometry, prepared beforehand
    // split-K tail: workgroup ids below main_tiles are whole tiles; the rest are `split` workgroups per tile that
    // each cover a slice of K and leave raw 128-bit partial sums in `partials`
    int main_tiles, split;
    int tail_xcd;                             // split tiles: deal (tile column, K slice) pairs over the 8 XCDs (see the kernel)
    int n_fastest;                            // tile order inside a batch: 0 = tile rows move fastest (the workgroups that run together share a B tile), 1 = tile columns (they share an A tile)
    unsigned long long *partials;
    int part64;                     // the partial sums fit 64 bits: only the low words are kept
    // grouped mode (GRP kernels): rows of A and C form one segment per group, each group has its own B.
    // Workgroup (mt, tn) looks up 32-row tile mt in grp_tiles = {group, first row} and stops at the segment's end.
    const int *grp_seg;             // [groups + 1] first row of every segment
    const int *grp_tiles;           // [2 * tiles] group and first row of every 32-row tile
    const int *grp_ntiles;          // how many of them exist (the grid is sized for the worst case)
    const void *const *grp_b;       // [groups] B of every group
    int b_shift;                    // BRS kernels: every element of B is divided by 2^b_shift first, truncating toward zero
    int finish_rq;                  // workgroups per tile of the finishing kernel (4 or 16)
    // guarded launches (the fallback behind a speculative launch): the kernel does nothing unless *guard is non-zero, and
    // its workgroups, one per compute unit, walk the `walk_blocks` workgroup ids of an ordinary launch
    const unsigned long long *guard;
    int walk_blocks;
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
__host__ __device__ static inline int limbs_needed(int64_t lo, int64_t hi)
{
    if (lo > hi) return 1;                   // nothing was seen
    for (int n = 1; n <= 8; n++) {
        // x + bias_n in [-2^(8n-1), 2^(8n-1))
        i128 bias = n == 1 ? 0 : (i128)(0x0080808080808080ull >> (8 * (8 - n)));
        i128 half = (i128)1 << (8 * n - 1);
        if ((i128)lo + bias >= -half && (i128)hi + bias < half) return n;
    }
    return 9;
}

// C++ division by 2^s (truncation toward zero) as shifts: the bias makes the arithmetic shift round negative values up
__device__ __forceinline__ int64_t tdiv_pow2(int64_t x, int s)
{
    const uint64_t bias = (uint64_t)(x >> 63) & (((uint64_t)1 << s) - 1);
    return (int64_t)((uint64_t)x + bias) >> s;
}

// ---- range tracking ------------------------------------------------------------------------------
struct MinMax { int64_t lo, hi; };

__device__ __forceinline__ void mm_update(MinMax &r, int64_t v)
{
    r.lo = v < r.lo ? v : r.lo;
    r.hi = v > r.hi ? v : r.hi;
}

// What the hot loop tracks instead of a 64-bit minimum and maximum (two quarter-rate compares and four selects per
// element; measured on the 512 x 7168 x 18432 product, 5.5 % of the kernel's time went into tracking B that way): the
// digit count itself.  In balanced base-256 digits x + 0x8080...80 has byte j equal to 0x80 wherever digit j is zero,
// so the OR over all elements of (x + 0x80..80) ^ 0x80..80 has its highest non-zero byte at the highest digit any
// element needs: six full-rate 32-bit instructions per element.  The range reported for n digits is the widest one n
// digits hold, [-0x80..80, 0x7F..7F] (n bytes each), which is all that the digit choice of the next call reads from it.
// (An element beyond eight digits wraps the sum; it leaves a non-zero top byte like one that needs eight, and both are
// reported as the full range: nine digits.)
struct DigitsSeen {
    uint32_t lo = 0, hi = 0;
    bool seen = false;
    __device__ __forceinline__ void add(int64_t v)
    {
        const uint64_t t = ((uint64_t)v + 0x8080808080808080ull) ^ 0x8080808080808080ull;
        lo |= (uint32_t)t;
        hi |= (uint32_t)(t >> 32);
    }
    __device__ __forceinline__ MinMax range() const
    {
        if (!seen) return MinMax{ INT64_MAX, INT64_MIN };
        const uint64_t e = ((uint64_t)hi << 32) | lo;
        if (e >> 56) return MinMax{ INT64_MIN, INT64_MAX };
        const int n = e ? (71 - __clzll((long long)e)) >> 3 : 1;          // bytes up to the highest non-zero one
        const uint64_t mask = ~0ull >> (64 - 8 * n);
        return MinMax{ -(int64_t)(0x8080808080808080ull & mask), (int64_t)(0x7F7F7F7F7F7F7F7Full & mask) };
    }
};

__device__ __forceinline__ void mm_merge(MinMax &r, const MinMax &o)
{
    r.lo = o.lo < r.lo ? o.lo : r.lo;
    r.hi = o.hi > r.hi ? o.hi : r.hi;
}

__device__ __forceinline__ MinMax mm_wave(MinMax r)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        int64_t ol = __shfl_xor(r.lo, off, kWave), oh = __shfl_xor(r.hi, off, kWave);
        r.lo = ol < r.lo ? ol : r.lo;
        r.hi = oh > r.hi ? oh : r.hi;
    }
    return r;
}

__device__ __forceinline__ void mm_publish(MinMax r, unsigned long long *slot)
{
    r = mm_wave(r);
    // The slots only ever move one way, so a plain (possibly stale) read is enough to skip the atomic when this
    // wave cannot improve them; that keeps thousands of waves from serialising on two addresses.
    if ((threadIdx.x & 63) == 0) {
        const unsigned long long lo = (unsigned long long)r.lo ^ kSignFlip, hi = (unsigned long long)r.hi ^ kSignFlip;
        if (lo < __atomic_load_n(slot, __ATOMIC_RELAXED)) atomicMin(slot, lo);
        if (hi > __atomic_load_n(slot + 1, __ATOMIC_RELAXED)) atomicMax(slot + 1, hi);
    }
}

static __global__ void range_reset_kernel(unsigned long long *range)
{
    if (threadIdx.x < 4) range[threadIdx.x] = (threadIdx.x & 1) ? 0ull : ~0ull;
}

// Strided sample of both operands for the first guess (at most `rows_s` rows x `cols_s` k each).
static __global__ __launch_bounds__(256) void range_sample_kernel(MfmaParams p, int b32, int G, int which)
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
                    v = tdiv_pow2(v, p.b_shift);
                }
                mm_update(r, v);
            }
        }
    }
    mm_publish(r, p.range + 2 * which);
}

// ---- element ownership ---------------------------------------------------------------------------
// Within a pipeline step of BK = 8*OCTS k-values, thread j (0 <= j < OCTS) of a row owns elements
//     k(e) = RUN*OCTS*(e / RUN) + RUN*j + e % RUN,   e = 0..7,
// i.e. 8/RUN runs of RUN consecutive k.  RUN = 2 for int64 B (a run is one 16-byte load), 4 for int32 B.
template <int RUN, int OCTS>
__device__ __forceinline__ int owned_k(int j, int e) { return RUN * OCTS * (e / RUN) + RUN * j + e % RUN; }

// Loads the 8 owned int64 elements of one row; `src` points at the row's first k of this step.
template <int RUN, int OCTS>
__device__ __forceinline__ void load_owned_i64(const int64_t *src_generic, int j, bool row_ok, int k_left, bool vec, int64_t (&x)[8])
{
    const ZK_GLOBAL_MEM int64_t *src = (const ZK_GLOBAL_MEM int64_t *)src_generic;
    if (row_ok && owned_k<RUN, OCTS>(j, 7) < k_left && vec) {
#pragma unroll
        for (int q = 0; q < 8 / RUN; q++) {
#pragma unroll
            for (int h = 0; h < RUN / 2; h++) {
                const v4i t = *(const ZK_GLOBAL_MEM v4i *)(src + owned_k<RUN, OCTS>(j, q * RUN + 2 * h));
                x[q * RUN + 2 * h] = (int64_t)(((uint64_t)(uint32_t)t[1] << 32) | (uint32_t)t[0]);
                x[q * RUN + 2 * h + 1] = (int64_t)(((uint64_t)(uint32_t)t[3] << 32) | (uint32_t)t[2]);
            }
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int k = owned_k<RUN, OCTS>(j, e);
            x[e] = (row_ok && k < k_left) ? src[k] : 0;
        }
    }
}

template <int RUN, int OCTS>
__device__ __forceinline__ void load_owned_i32(const int32_t *src_generic, int j, bool row_ok, int k_left, bool vec, int64_t (&x)[8])
{
    const ZK_GLOBAL_MEM int32_t *src = (const ZK_GLOBAL_MEM int32_t *)src_generic;
    if (RUN == 4 && row_ok && owned_k<RUN, OCTS>(j, 7) < k_left && vec) {
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const v4i t = *(const ZK_GLOBAL_MEM v4i *)(src + owned_k<RUN, OCTS>(j, q * 4));
#pragma unroll
            for (int z = 0; z < 4; z++) x[q * 4 + z] = (int64_t)t[z];
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int k = owned_k<RUN, OCTS>(j, e);
            x[e] = (row_ok && k < k_left) ? (int64_t)src[k] : 0;
        }
    }
}

// Byte offset, inside one operand region of an LDS stage (or of a plane step), of the 8 digit bytes that
// thread j of `row` produces: 1 KB fragment blocks, lane slot = row%32 + 32*(k-half), 16 bytes per slot.
__device__ __forceinline__ int frag_offset(int row, int j, int n_limbs, int substage_bytes)
{
    const int o4 = j & 3;
    return (j >> 2) * substage_bytes + ((row >> 5) * n_limbs) * 1024 + ((row & 31) + 32 * (o4 >> 1)) * 16 + (o4 & 1) * 8;
}

// ---- A digit planes (pre-pass) ------------------------------------------------------------------
// When A is reused by many column tiles it is split once, into digit planes stored in MFMA fragment order:
// block (g, sub, ks32, i) of 1 KB holds digit i of rows [32*sub, 32*sub+32) for the 32 owned-k slots of MFMA
// depth ks32, lane-major.  Rows >= M and k >= K are written as zero digits.  Each workgroup also leaves the
// min and max of what it read in mm[2*block .. 2*block+1].
// IN32: the matrix holds int32 elements (weights prepared once; lda and sA count elements as they do for int64).
template <int NA, int RUN, int KK, bool IN32 = false>
__global__ __launch_bounds__(256) void a_planes_kernel(MfmaParams p, unsigned char *planes, int msub, int ksteps32,
                                                       unsigned long long *mm)
{
    constexpr int OCTS = 4 * KK, ROWS = 256 / OCTS;
    __shared__ MinMax red[4];
    const int tid = threadIdx.x;
    const int g = blockIdx.z, ks = blockIdx.x;
    const int row = blockIdx.y * ROWS + tid / OCTS, j = tid % OCTS;
    const int k0 = ks * (8 * OCTS);
    const bool vec = (((uintptr_t)p.A | (uintptr_t)(p.lda * 8) | (uintptr_t)(p.sA * 8)) & 15) == 0;
    int64_t x[8];
    if (IN32) load_owned_i32<RUN, OCTS>(reinterpret_cast<const int32_t *>(p.A) + (long)g * p.sA + (long)row * p.lda + k0, j, row < p.M, p.K - k0, false, x);
    else load_owned_i64<RUN, OCTS>(p.A + (long)g * p.sA + (long)row * p.lda + k0, j, row < p.M, p.K - k0, vec, x);
    DigitsSeen bound;
#pragma unroll
    for (int q = 0; q < 8; q++) bound.add(x[q]);
    bound.seen = true;
    MinMax r = bound.range();
    uint2 dg[NA];
    limb_split8<NA>(x, dg);
    // plane step layout: [g][sub][ks32][digit][1 KB]; a step of KK depths is contiguous per sub
    unsigned char *dst = planes + (((long)g * msub + (row >> 5)) * ksteps32 + ks * KK + (j >> 2)) * (NA * 1024) +
                         ((row & 31) + 32 * ((j & 3) >> 1)) * 16 + (j & 1) * 8;
    if (row < msub * 32) {                  // a workgroup may reach past the last 32-row group (skinny tiles)
#pragma unroll
        for (int i = 0; i < NA; i++) *reinterpret_cast<uint2 *>(dst + i * 1024) = dg[i];
    }
    r = mm_wave(r);
    if ((tid & 63) == 0) red[tid >> 6] = r;
    __syncthreads();
    if (tid == 0) {
#pragma unroll
        for (int w = 1; w < 4; w++) mm_merge(r, red[w]);
        const long b = ((long)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
        mm[2 * b] = (unsigned long long)r.lo ^ kSignFlip;
        mm[2 * b + 1] = (unsigned long long)r.hi ^ kSignFlip;
    }
}

// Folds the per-workgroup ranges of the plane pre-pass (`mm`, A only) and of the GEMM kernel (`wg`, A and B) into
// range[0..3] and leaves the verdict in range[4]: 0 when `na` and `nb` digits covered them, otherwise 1 when five digits
// cover both operands and 2 when they do not (what the guarded launch behind the product multiplies with).
// `host_copy`, when set, is pinned host memory that receives the same five words.
// `parts` workgroups (of any size) share the slots; each leaves its partial result in `scratch` and takes a ticket, and
// the one that arrives last folds the partials (a launch with tens of thousands of tiles would otherwise spend longer
// in a one-workgroup fold than some GEMMs take).  range[5] is the ticket counter; it is zero between launches.
constexpr int kFoldParts = 64;        // at most this many workgroups fold
constexpr long kFoldSlotsPerPart = 1024;

struct FoldArgs {
    const unsigned long long *mm;
    long mm_count;
    const unsigned long long *wg;
    long wg_count;
    unsigned long long *range;
    int na, nb;
    unsigned long long *host_copy;
    int parts;
    unsigned long long *scratch;      // 4 * kFoldParts words
};

__host__ __device__ inline unsigned long long fold_pick(int q, unsigned long long a, unsigned long long b)
{
    return (q & 1) ? (a > b ? a : b) : (a < b ? a : b);       // words 1 and 3 are maxima, 0 and 2 minima
}

__device__ __forceinline__ void range_fold_body(const FoldArgs &f, int part)
{
    __shared__ unsigned long long red[16][4];
    const int nthreads = blockDim.x;
    const long first = (long)part * nthreads + threadIdx.x, stride = (long)f.parts * nthreads;
    unsigned long long v[4] = { ~0ull, 0ull, ~0ull, 0ull };
    for (long i = first; i < f.mm_count; i += stride) {
        v[0] = fold_pick(0, f.mm[2 * i], v[0]);
        v[1] = fold_pick(1, f.mm[2 * i + 1], v[1]);
    }
    for (long i = first; i < f.wg_count; i += stride) {
#pragma unroll
        for (int q = 0; q < 4; q++) v[q] = fold_pick(q, f.wg[4 * i + q], v[q]);
    }
#pragma unroll
    for (int q = 0; q < 4; q++) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1)
            v[q] = fold_pick(q, (unsigned long long)__shfl_xor((long long)v[q], off, kWave), v[q]);
    }
    if ((threadIdx.x & 63) == 0) {
#pragma unroll
        for (int q = 0; q < 4; q++) red[threadIdx.x >> 6][q] = v[q];
    }
    __syncthreads();
    if (threadIdx.x != 0) return;
    for (int w = 1; w < nthreads / 64; w++)
#pragma unroll
        for (int q = 0; q < 4; q++) v[q] = fold_pick(q, red[w][q], v[q]);
    if (f.parts > 1) {
#pragma unroll
        for (int q = 0; q < 4; q++) __hip_atomic_store(&f.scratch[4 * part + q], v[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // release the partial, then count in; whoever sees everyone else counted in acquires their partials
        const unsigned long long ticket = __hip_atomic_fetch_add(&f.range[5], 1ull, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        if (ticket != (unsigned long long)(f.parts - 1)) return;
        for (int w = 0; w < f.parts; w++)
#pragma unroll
            for (int q = 0; q < 4; q++)
                v[q] = fold_pick(q, __hip_atomic_load(&f.scratch[4 * w + q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), v[q]);
        __hip_atomic_store(&f.range[5], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int q = 0; q < 4; q++) f.range[q] = v[q];
    const int need_a = limbs_needed((int64_t)(v[0] ^ kSignFlip), (int64_t)(v[1] ^ kSignFlip));
    const int need_b = limbs_needed((int64_t)(v[2] ^ kSignFlip), (int64_t)(v[3] ^ kSignFlip));
    const unsigned long long verdict = (need_a <= f.na && need_b <= f.nb) ? 0ull : ((need_a <= 5 && need_b <= 5) ? 1ull : 2ull);
    f.range[4] = verdict;
    if (f.host_copy) {
#pragma unroll
        for (int q = 0; q < 4; q++) f.host_copy[q] = v[q];
        f.host_copy[4] = verdict;
    }
}

static __global__ __launch_bounds__(256) void range_fold_kernel(FoldArgs f) { range_fold_body(f, (int)blockIdx.x); }

// Number of digit pairs (i', j') with i' + j' < d that come before (i, j) in row order (i' < i, or i' == i and j' < j).
__host__ __device__ constexpr int kept_pairs_before(int na, int nb, int d, int i, int j)
{
    int n = 0;
    for (int r = 0; r < i && r < na; r++) {
        const int row = d - r < 0 ? 0 : (d - r > nb ? nb : d - r);
        n += row;
    }
    if (i < na) {
        const int row = d - i < 0 ? 0 : (d - i > nb ? nb : d - i);
        n += j < row ? j : row;
    }
    return n;
}

// ---- the GEMM kernel -------------------------------------------------------------------------------
// WVM x WVN waves per workgroup, WM x WN 32x32 MFMA tiles per wave, KK MFMA k-depths (32 k each) per pipeline
// step.  APL: A comes from pre-split digit planes (plain copy into LDS); otherwise it is split on the fly like B.
// BPL: so does B (weights prepared once, in the layout of the A planes with columns for rows); nothing of B is tracked then,
// its digit count was fixed exactly when the planes were made.
//
// The hot loop is branch-free: rows past M or N are clamped to the last valid row (their products land in
// outputs that are never stored), only a final partial k-step uses guarded loads, and every thread walks its
// own row pointers.  Loads of step s+1 are issued first, the MFMAs of the step's leading depths give them time
// to land, and the MFMAs of the last depth are interleaved with the digit split of the loaded data.
// (the body of the kernels below: `block` is the workgroup id of an ordinary launch, one tile or one slice of a split tile)
template <int NA, int NB, int WVM, int WVN, int WM, int WN, int KK, bool B32, bool BKM, bool APL, bool GRP = false, bool BRS = false, int DMAX = 16,
          bool BPL = false>
__device__ __forceinline__ void gemm_mfma_block(const MfmaParams &p, const int block)
{
    constexpr int T = 64 * WVM * WVN;
    constexpr int BM = 32 * WM * WVM, BN = 32 * WN * WVN, BK = 32 * KK, OCTS = BK / 8;
    constexpr int RUN = B32 ? 4 : 2;
    // Diagonal d carries weight 2^(8d).  Diagonal 16 (2^128) never matters; a launch whose shift + 64 result bits
    // end below 2^(8 DMAX) leaves out the digit pairs of the diagonals from DMAX up as well.
    constexpr int D = (NA + NB - 1) > DMAX ? DMAX : (NA + NB - 1);
    static_assert(DMAX >= 8 && DMAX <= 16, "the low 64 bits of the sum need diagonals 0..7");
    constexpr int A_BLOCKS = (BM / 32) * NA, B_BLOCKS = (BN / 32) * NB;
    constexpr int SUBSTAGE = (A_BLOCKS + B_BLOCKS) * 1024;
    constexpr int STAGE = KK * SUBSTAGE;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WVN, wn = wave % WVN;

    // workgroup -> tile.  Consecutive workgroup ids go to different XCDs (8 of them, each with its own L2), so
    // ids are regrouped to give each XCD a contiguous run of tiles; within a run the tile-row index moves
    // fastest, so the workgroups that share a B tile sit on the same L2.
    const int per_batch = p.tiles_m * p.tiles_n;
    int lin = block, sidx = 0, nsplit = 1;
    int tail_tile = 0, g = 0, tn, tm, m0, m_lim = p.M;
    const void *b_base = p.B;
    if (GRP) {
        // Consecutive workgroup ids go round the 8 XCDs, each with its own L2: the tile columns of one 32-row tile go to
        // ONE of them, so that its rows of A come from memory once and not once per tile column (the routed experts'
        // w1/w3 launch fetched 15.68 GB for 14.86 that way).  The grid is a multiple of 8 * tiles_n workgroups.
        const int xcd = lin & 7, w = lin >> 3, wq = w / p.tiles_n;
        const int mt = wq * 8 + xcd;
        if (mt >= *p.grp_ntiles) {                 // the grid covers the worst case: nothing to do, an empty range
            if (tid == 0) {
                unsigned long long *slot = p.wg_range + 4 * (long)block;
                slot[0] = ~0ull; slot[1] = 0ull; slot[2] = ~0ull; slot[3] = 0ull;
            }
            return;
        }
        tn = w - wq * p.tiles_n;
        tm = 0;
        const int e = p.grp_tiles[2 * mt];
        m0 = p.grp_tiles[2 * mt + 1];
        m_lim = p.grp_seg[e + 1];
        b_base = p.grp_b[e];
    } else {
        if (lin < p.main_tiles) {
            if ((p.main_tiles & 7) == 0) lin = (lin & 7) * (p.main_tiles >> 3) + (lin >> 3);
        } else {
            const int t = lin - p.main_tiles;
            if (p.tail_xcd) {
                // Workgroup ids go round the 8 XCDs.  Each XCD takes whole (tile column, K slice) pairs and runs the
                // tiles_m workgroups of a pair one after the other, so that they find the pair's B data in their L2.
                const int x = t & 7, q = t >> 3;
                const int pair = (q / p.tiles_m) * 8 + x;
                lin = p.main_tiles + (pair / p.split) * p.tiles_m + q % p.tiles_m;
                sidx = pair % p.split;
            } else {
                lin = p.main_tiles + t / p.split;
                sidx = t % p.split;
            }
            nsplit = p.split;
        }
        tail_tile = lin - p.main_tiles;            // index among the split tiles (when nsplit > 1)
        g = lin / per_batch;
        const int rem = lin - g * per_batch;
        if (p.n_fastest) { tm = rem / p.tiles_n; tn = rem - tm * p.tiles_n; }
        else { tn = rem / p.tiles_m; tm = rem - tn * p.tiles_m; }
        m0 = tm * BM;
    }
    const int n0 = tn * BN;

    // Range tracking is shared out: the tiles_m workgroups that load the same B tile each check every
    // tiles_m-th k-step of it (likewise for A across the workgroups of a tile row), so no workgroup is slower
    // than its neighbours and every element is still seen once.
    const int vmod_b = p.tiles_m < 8 ? p.tiles_m : 8, vmod_a = p.tiles_n < 8 ? p.tiles_n : 8;
    const bool verify_a = !APL && tn < vmod_a;
    const bool verify_b = !BPL && tm < vmod_b && (g == 0 || p.verify_b_all_batches);
    DigitsSeen oa, ob;
    int rb32_lo = INT32_MAX, rb32_hi = INT32_MIN;        // the range of an int32 B is tracked in 32 bits and joins rb at the end

    v16i acc[WM][WN][D];
#pragma unroll
    for (int a = 0; a < WM; a++)
#pragma unroll
        for (int b = 0; b < WN; b++)
#pragma unroll
            for (int d = 0; d < D; d++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[a][b][d][r] = 0;

    // Work items of the loaders: (row, j) pairs owning 8 elements each, or 16-byte chunks of digit planes.
    constexpr int A_ITEMS = BM * OCTS, B_ITEMS = BN * OCTS;
    constexpr int A_IT = APL ? 1 : (A_ITEMS + T - 1) / T, B_IT = BPL ? 1 : (B_ITEMS + T - 1) / T;
    constexpr int A_CHUNKS = KK * A_BLOCKS * 64, A_CIT = APL ? (A_CHUNKS + T - 1) / T : 1;
    constexpr int B_CHUNKS = KK * B_BLOCKS * 64, B_CIT = BPL ? (B_CHUNKS + T - 1) / T : 1;
    static_assert(!BPL || (!B32 && !BKM && !BRS), "prepared planes of B go with the int64 forms (and are made for the kernel's KK: the owned-k order depends on it)");
    int64_t sa[A_IT][8], sb[B_IT][8];
    v4i pa[A_CIT], pb[B_CIT];

    const bool a_vec = (((uintptr_t)p.A | (uintptr_t)(p.lda * 8) | (uintptr_t)(p.sA * 8)) & 15) == 0;
    const bool b_vec = BPL || (!BKM && (((uintptr_t)b_base | (uintptr_t)(p.ldbn * (B32 ? 4 : 8)) | (uintptr_t)(p.sB * (B32 ? 4 : 8))) & 15) == 0);

    // per-thread source pointers (advanced by BK per step) and LDS destinations
    const int64_t *a_src[A_IT];
    const unsigned char *a_pl[A_CIT];
    const char *b_src[B_IT];
    const unsigned char *b_pl[B_CIT];
    // LDS destinations are stage-relative; threads with no work in an iteration aim at a dummy area behind the two
    // stages (and a zero stage stride), which keeps the loop body free of branches.
    constexpr int DUMMY = 2 * STAGE;
    bool a_pad[A_IT];
    int a_j[A_IT], b_j[B_IT], a_dst[A_IT], b_dst[B_IT], pl_dst[A_CIT], plb_dst[B_CIT];
    int a_stride[A_IT], b_stride[B_IT], pl_stride[A_CIT], plb_stride[B_CIT];
    if (APL) {
#pragma unroll
        for (int it = 0; it < A_CIT; it++) {
            const int c = it * T + tid;
            const bool live = A_CHUNKS % T == 0 || c < A_CHUNKS;
            const int cc0 = live ? c : 0;
            // LDS order inside a stage is [kk][sub][digit]; planes are [sub][ks32][digit]
            const int kk = cc0 / (A_BLOCKS * 64), cc = cc0 - kk * (A_BLOCKS * 64);
            const int sub_i = cc / (NA * 64), within = cc - sub_i * (NA * 64);
            a_pl[it] = p.a_planes + (((long)g * p.a_msub + (m0 >> 5) + sub_i) * p.a_ksteps + kk) * (NA * 1024) + within * 16;
            pl_dst[it] = live ? kk * SUBSTAGE + cc * 16 : DUMMY;
            pl_stride[it] = live ? STAGE : 0;
        }
    } else {
#pragma unroll
        for (int it = 0; it < A_IT; it++) {
            const int idx = it * T + tid;
            const bool live = A_ITEMS % T == 0 || idx < A_ITEMS;
            const int row = (live ? idx : 0) / OCTS;
            a_j[it] = idx % OCTS;
            int m = m0 + row;
            // (rows past the end are loaded from the last row, a valid address, and multiplied as zeros: the device is
            // power managed and what the matrix pipe draws depends on the bits it is fed; an expert's tile has some
            // 8 real rows of 32)
            a_pad[it] = m >= m_lim;
            m = m < m_lim ? m : m_lim - 1;
            a_src[it] = p.A + (long)g * p.sA + (long)m * p.lda;
            a_dst[it] = live ? frag_offset(row, a_j[it], NA, SUBSTAGE) : DUMMY;
            a_stride[it] = live ? STAGE : 0;
        }
    }
    if (BPL) {
#pragma unroll
        for (int it = 0; it < B_CIT; it++) {
            const int c = it * T + tid;
            const bool live = B_CHUNKS % T == 0 || c < B_CHUNKS;
            const int cc0 = live ? c : 0;
            // as for the planes of A: LDS order inside a stage is [kk][sub][digit], planes are [sub][ks32][digit]
            const int kk = cc0 / (B_BLOCKS * 64), cc = cc0 - kk * (B_BLOCKS * 64);
            const int sub_i = cc / (NB * 64), within = cc - sub_i * (NB * 64);
            int sub = (n0 >> 5) + sub_i;
            sub = sub < p.b_nsub ? sub : p.b_nsub - 1;          // column groups past N: any valid data, never stored
            b_pl[it] = reinterpret_cast<const unsigned char *>(b_base) + ((long)sub * p.b_ksteps + kk) * (NB * 1024) + within * 16;
            plb_dst[it] = live ? A_BLOCKS * 1024 + kk * SUBSTAGE + cc * 16 : DUMMY;
            plb_stride[it] = live ? STAGE : 0;
        }
    }
#pragma unroll
    for (int it = 0; it < (BPL ? 0 : B_IT); it++) {
        const int idx = it * T + tid;
        const bool live = B_ITEMS % T == 0 || idx < B_ITEMS;
        const int idx0 = live ? idx : 0;
        int row;
        if (BKM) { row = (idx0 & 63) + 64 * (idx0 / (64 * OCTS)); b_j[it] = (idx0 >> 6) % OCTS; }
        else { row = idx0 / OCTS; b_j[it] = idx0 % OCTS; }
        int n = n0 + row;
        n = n < p.N ? n : p.N - 1;
        const long off = (long)g * p.sB + (long)n * p.ldbn;
        b_src[it] = reinterpret_cast<const char *>(b_base) + off * (B32 ? 4 : 8);
        b_dst[it] = live ? A_BLOCKS * 1024 + frag_offset(row, b_j[it], NB, SUBSTAGE) : DUMMY;
        b_stride[it] = live ? STAGE : 0;
    }

    // The staged data of a step can be handled in two parts, so that a kernel with two MFMA depths per step splits,
    // stores and reloads one half behind each depth (its loads are then spread over the step instead of leaving in one
    // burst at its end): PART 0 = A and the first half of B's items, 1 = the rest of B, -1 = everything.
    typedef std::integral_constant<int, -1> PAll;
    typedef std::integral_constant<int, 0> PFirst;
    typedef std::integral_constant<int, 1> PSecond;
    constexpr int B_N = BPL ? B_CIT : B_IT;          // items (or chunks of planes) of B per thread

    // FAST: the whole step lies inside K and the pointers allow 16-byte loads: no guards at all.
    auto fetch = [&](int ks, auto fast_tag, auto part_tag) {
        constexpr bool FAST = decltype(fast_tag)::value;
        constexpr int PART = decltype(part_tag)::value;
        constexpr int B_LO = PART == 1 ? B_N / 2 : 0, B_HI = PART == 0 ? B_N / 2 : B_N;
        const int k0 = ks * BK;
        if (PART == 1) {
        } else if (APL) {
#pragma unroll
            for (int it = 0; it < A_CIT; it++)
                pa[it] = *reinterpret_cast<const v4i *>(a_pl[it] + (long)ks * (KK * NA * 1024));
        } else {
#pragma unroll
            for (int it = 0; it < A_IT; it++) {
                if (FAST) load_owned_i64<RUN, OCTS>(a_src[it] + k0, a_j[it], true, BK, true, sa[it]);
                else load_owned_i64<RUN, OCTS>(a_src[it] + k0, a_j[it], true, p.K - k0, false, sa[it]);
            }
        }
        if (BPL) {
#pragma unroll
            for (int it = B_LO; it < B_HI; it++)
                pb[it] = *(const ZK_GLOBAL_MEM v4i *)(b_pl[it] + (long)ks * (KK * NB * 1024));
        }
#pragma unroll
        for (int it = (BPL ? 0 : B_LO); it < (BPL ? 0 : B_HI); it++) {
            if (BKM) {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int k = k0 + owned_k<RUN, OCTS>(b_j[it], e);
                    const long off = (long)k * p.ldbk;
                    int64_t v = 0;
                    if (FAST || k < p.K)
                        v = B32 ? (int64_t)((const ZK_GLOBAL_MEM int32_t *)b_src[it])[off] : ((const ZK_GLOBAL_MEM int64_t *)b_src[it])[off];
                    sb[it][e] = v;
                }
            } else if (B32) {
                const int32_t *src = reinterpret_cast<const int32_t *>(b_src[it]) + k0;
                if (FAST) load_owned_i32<RUN, OCTS>(src, b_j[it], true, BK, true, sb[it]);
                else load_owned_i32<RUN, OCTS>(src, b_j[it], true, p.K - k0, false, sb[it]);
            } else {
                const int64_t *src = reinterpret_cast<const int64_t *>(b_src[it]) + k0;
                if (FAST) load_owned_i64<RUN, OCTS>(src, b_j[it], true, BK, true, sb[it]);
                else load_owned_i64<RUN, OCTS>(src, b_j[it], true, p.K - k0, false, sb[it]);
            }
        }
    };

    // staged elements -> digits -> LDS stage `buf`, fragment order
    auto stash = [&](int buf, auto part_tag) {
        constexpr int PART = decltype(part_tag)::value;
        constexpr int B_LO = PART == 1 ? B_N / 2 : 0, B_HI = PART == 0 ? B_N / 2 : B_N;
        if (PART == 1) {
        } else if (APL) {
#pragma unroll
            for (int it = 0; it < A_CIT; it++)
                *reinterpret_cast<v4i *>(smem + pl_dst[it] + buf * pl_stride[it]) = pa[it];
        } else {
#pragma unroll
            for (int it = 0; it < A_IT; it++) {
                uint2 dg[NA];
                limb_split8<NA>(sa[it], dg);
#pragma unroll
                for (int i = 0; i < NA; i++)
                    *reinterpret_cast<uint2 *>(smem + a_dst[it] + buf * a_stride[it] + i * 1024) = a_pad[it] ? make_uint2(0u, 0u) : dg[i];
            }
        }
        if (BPL) {
#pragma unroll
            for (int it = B_LO; it < B_HI; it++)
                *reinterpret_cast<v4i *>(smem + plb_dst[it] + buf * plb_stride[it]) = pb[it];
        }
#pragma unroll
        for (int it = (BPL ? 0 : B_LO); it < (BPL ? 0 : B_HI); it++) {
            uint2 dg[NB];
            if (BRS) {
                int64_t y[8];
#pragma unroll
                for (int q = 0; q < 8; q++) y[q] = tdiv_pow2(sb[it][q], p.b_shift);
                limb_split8<NB>(y, dg);
            } else {
                limb_split8<NB>(sb[it], dg);
            }
#pragma unroll
            for (int i = 0; i < NB; i++)
                *reinterpret_cast<uint2 *>(smem + b_dst[it] + buf * b_stride[it] + i * 1024) = dg[i];
        }
    };

    // Fragments of one MFMA depth, and the MFMAs of a slice [LO, HI) of the depth's (i, j, tile) list.
    auto load_frags = [&](int buf, int kk, v4i (&fa)[WM][NA], v4i (&fb)[WN][NB]) {
        const unsigned char *base = smem + buf * STAGE + kk * SUBSTAGE;
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
    };
    // the digit pairs (i, j) with i + j < D are numbered in row order; a slice issues those numbered LO..HI-1
    constexpr int MFMAS = WM * WN * kept_pairs_before(NA, NB, D, NA, 0);
    auto mfma_slice = [&](auto lo_tag, auto hi_tag, const v4i (&fa)[WM][NA], const v4i (&fb)[WN][NB]) {
        constexpr int LO = decltype(lo_tag)::value, HI = decltype(hi_tag)::value;
#pragma unroll
        for (int i = 0; i < NA; i++)
#pragma unroll
            for (int j = 0; j < NB; j++)
#pragma unroll
                for (int a = 0; a < WM; a++)
#pragma unroll
                    for (int b = 0; b < WN; b++) {
                        const int idx = (kept_pairs_before(NA, NB, D, i, j) * WM + a) * WN + b;
                        if (idx >= LO && idx < HI && i + j < D)
                            acc[a][b][i + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[a][i], fb[b][j], acc[a][b][i + j], 0, 0, 0);
                    }
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, MFMAS / 2> IH;
    typedef std::integral_constant<int, MFMAS> IF;
    auto compute_all = [&](int buf) {
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
            v4i fa[WM][NA], fb[WN][NB];
            load_frags(buf, kk, fa, fb);
            mfma_slice(I0(), IF(), fa, fb);
        }
    };

    const int ksteps = (p.K + BK - 1) / BK;
    const int full_steps = (a_vec || APL) && (b_vec || BKM) ? p.K / BK : 0;     // steps that can use unguarded loads
    // this workgroup's slice of the k-steps (everything unless it is one of the split workgroups of a tail tile)
    const int ks_begin = (int)((long)sidx * ksteps / nsplit), ks_end = (int)((long)(sidx + 1) * ksteps / nsplit);

    // Range tracking of the staged elements of data step d, done while the registers still hold them.
    // (called once per data step, in order: the turn counters stand for d % vmod_a and d % vmod_b without a division)
    int turn_a = ks_begin % vmod_a, turn_b = ks_begin % vmod_b;
    bool my_a = false, my_b = false;
    auto track = [&](auto part_tag) {
        constexpr int PART = decltype(part_tag)::value;
        constexpr int B_LO = PART == 1 ? B_IT / 2 : 0, B_HI = PART == 0 ? B_IT / 2 : B_IT;
        if (PART != 1) {            // (the turns advance once per data step, with its first part)
            my_a = turn_a == tn;
            my_b = turn_b == tm;
            turn_a = turn_a + 1 == vmod_a ? 0 : turn_a + 1;
            turn_b = turn_b + 1 == vmod_b ? 0 : turn_b + 1;
        }
        if (PART != 1 && verify_a && my_a) {
#pragma unroll
            for (int it = 0; it < A_IT; it++)
#pragma unroll
                for (int q = 0; q < 8; q++) oa.add(sa[it][q]);
            oa.seen = true;
        }
        if (verify_b && my_b) {
#pragma unroll
            for (int it = B_LO; it < B_HI; it++)
#pragma unroll
                for (int q = 0; q < 8; q++) {
                    if (B32 && !BRS) {
                        // int32 values: one min and one max instruction each, against four for a 64-bit pair
                        const int v = (int)sb[it][q];
                        rb32_lo = v < rb32_lo ? v : rb32_lo;
                        rb32_hi = v > rb32_hi ? v : rb32_hi;
                    } else {
                        ob.add(BRS ? tdiv_pow2(sb[it][q], p.b_shift) : sb[it][q]);     // what the digits are taken from
                    }
                }
            ob.seen = true;
        }
    };

    // One pipeline step, three fenced phases:
    //   A  fragment reads of stage `cur` and the first half of its MFMAs (time for the staged loads to land);
    //   B  the second half of the MFMAs interleaved, in one scheduling region, with the digit split of the
    //      elements staged for step ks+1 and their LDS writes into the other stage;
    //   C  the loads of step ks+2 into the now free staging registers, then the barrier.
    // Two depths per step, B split on the fly: one depth's MFMAs carry the split of one half of the staged data, whose
    // registers are reloaded right behind it.  Each half's loads then have a whole step to land and some are under way
    // at every moment (with one burst per step nothing is for the part of the step between their arrival and the next
    // burst: the routed experts' int32 weights streamed at 5.3 TB/s that way).
    constexpr bool SPREAD = KK == 2 && !BKM && B_N >= 2 && B_N % 2 == 0;
    auto step_body = [&](int ks, auto fast_tag) {
        const int cur = (ks - ks_begin) & 1;
        if constexpr (SPREAD) {
            {
                v4i fa[WM][NA], fb[WN][NB];
                load_frags(cur, 0, fa, fb);
                mfma_slice(I0(), IF(), fa, fb);
                stash(cur ^ 1, PFirst());
#pragma unroll
                for (int i = 0; i < MFMAS; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, ZK_VALU_PER_MFMA, 0);
                    __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                track(PFirst());
                if (ks + 2 < ks_end) fetch(ks + 2, fast_tag, PFirst());
                __builtin_amdgcn_sched_barrier(0);
            }
            {
                v4i fa[WM][NA], fb[WN][NB];
                load_frags(cur, 1, fa, fb);
                mfma_slice(I0(), IF(), fa, fb);
                stash(cur ^ 1, PSecond());
#pragma unroll
                for (int i = 0; i < MFMAS; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, ZK_VALU_PER_MFMA, 0);
                    __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                track(PSecond());
                if (ks + 2 < ks_end) fetch(ks + 2, fast_tag, PSecond());
            }
            __syncthreads();
            return;
        }
#pragma unroll
        for (int kk = 0; kk < KK - 1; kk++) {
            v4i fa[WM][NA], fb[WN][NB];
            load_frags(cur, kk, fa, fb);
            mfma_slice(I0(), IF(), fa, fb);
        }
        v4i fa[WM][NA], fb[WN][NB];
        load_frags(cur, KK - 1, fa, fb);
        mfma_slice(I0(), IH(), fa, fb);
        __builtin_amdgcn_sched_barrier(0);
        mfma_slice(IH(), IF(), fa, fb);
        stash(cur ^ 1, PAll());
#pragma unroll
        for (int i = 0; i < MFMAS - MFMAS / 2; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, ZK_VALU_PER_MFMA, 0);
            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        track(PAll());
        if (ks + 2 < ks_end) fetch(ks + 2, fast_tag, PAll());
        __syncthreads();
    };

    // prologue: stage 0 holds the first step, the staging registers hold the second
    if (ks_begin < full_steps) fetch(ks_begin, std::true_type(), PAll()); else fetch(ks_begin, std::false_type(), PAll());
    track(PAll());
    stash(0, PAll());
    if (ks_begin + 1 < ks_end) {
        if (ks_begin + 1 < full_steps) fetch(ks_begin + 1, std::true_type(), PAll()); else fetch(ks_begin + 1, std::false_type(), PAll());
    }
    __syncthreads();
    int ks = ks_begin;
    const int fast_end = full_steps < ks_end ? full_steps : ks_end;
    for (; ks + 2 < fast_end; ks++) step_body(ks, std::true_type());
    for (; ks + 1 < ks_end; ks++) step_body(ks, std::false_type());
    compute_all((ks_end - 1 - ks_begin) & 1);

    // every workgroup leaves its ranges (empty ones included) in its own slot; the waves' ranges meet in LDS
    // (the stages are free by now)
    MinMax ra = { INT64_MAX, INT64_MIN }, rb = { INT64_MAX, INT64_MIN };
    if (verify_a || verify_b) {
        __syncthreads();
        MinMax *red = reinterpret_cast<MinMax *>(smem);
        ra = oa.range();
        rb = ob.range();
        if (B32 && !BRS && rb32_lo <= rb32_hi) mm_merge(rb, MinMax{ (int64_t)rb32_lo, (int64_t)rb32_hi });
        ra = mm_wave(ra);
        rb = mm_wave(rb);
        if (lane == 0) { red[2 * wave] = ra; red[2 * wave + 1] = rb; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < T / 64; w++) { mm_merge(ra, red[2 * w]); mm_merge(rb, red[2 * w + 1]); }
        }
    }
    if (tid == 0) {
        unsigned long long *slot = p.wg_range + 4 * (long)block;
        slot[0] = (unsigned long long)ra.lo ^ kSignFlip;
        slot[1] = (unsigned long long)ra.hi ^ kSignFlip;
        slot[2] = (unsigned long long)rb.lo ^ kSignFlip;
        slot[3] = (unsigned long long)rb.hi ^ kSignFlip;
    }

    // epilogue: diagonals -> 128-bit sum -> shift.  Accumulator register r of lane l holds
    // row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its 32x32 tile.
    // Diagonals are added in groups of four: a group's sum of v[4g+j] * 2^(8j) stays below 2^57, so it is plain 64-bit
    // arithmetic; the groups (weights 2^0, 2^32, 2^64, 2^96) then meet in one 128-bit sum.
    auto combine = [&](int a, int b, int r, u128 sum) {
#pragma unroll
        for (int gq = 0; gq < (D + 3) / 4; gq++) {
            uint64_t s = (uint64_t)(int64_t)acc[a][b][4 * gq][r];
#pragma unroll
            for (int j = 1; j < 4; j++)
                if (4 * gq + j < D) s += (uint64_t)(int64_t)acc[a][b][4 * gq + j][r] << (8 * j);
            sum += (u128)(i128)(int64_t)s << (32 * gq);
        }
        return sum;
    };
    if (nsplit > 1) {
        // raw partial sums (without the rounding term), finished by gemm_split_finish_kernel: 64 lanes' low words, then
        // (unless 64 bits hold the sums) their high words, per (slice, wave, tile, register)
#pragma unroll
        for (int a = 0; a < WM; a++)
#pragma unroll
            for (int b = 0; b < WN; b++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    // rows of this register that all lie past M (uniform over the wave): nothing to keep
                    if (m0 + (wm * WM + a) * 32 + 8 * (r >> 2) + (r & 3) >= m_lim) continue;
                    const u128 sum = combine(a, b, r, 0);
                    const long q = (((long)tail_tile * p.split + sidx) * (T / 64) + wave) * (WM * WN * 16) + (a * WN + b) * 16 + r;
                    if (p.part64) p.partials[q * 64 + lane] = (uint64_t)sum;
                    else { p.partials[q * 128 + lane] = (uint64_t)sum; p.partials[q * 128 + 64 + lane] = (uint64_t)(sum >> 64); }
                }
        return;
    }
    // Whole tiles: the loops carry no uniform branches (tiles that reach past M or N, and calls that want the remainder,
    // have their own copy), and a row's address is the tile's plus a scalar multiple of the row stride.
    const uint64_t rmask = p.shift ? ((1ull << p.shift) - 1) : 0;
    const u128 sum0 = (u128)(i128)p.init;
    const int sh = p.shift;
    auto store_tile = [&](auto edge_tag, auto rem_tag) {
        constexpr bool EDGE = decltype(edge_tag)::value, REM = decltype(rem_tag)::value;
#pragma unroll
        for (int a = 0; a < WM; a++)
#pragma unroll
            for (int b = 0; b < WN; b++) {
                const int n = n0 + (wn * WN + b) * 32 + (lane & 31);
                const int mrow = m0 + (wm * WM + a) * 32 + 4 * (lane >> 5);
                const long o0 = (long)g * p.sC + (long)mrow * p.ldc + n;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int dr = 8 * (r >> 2) + (r & 3);
                    const u128 sum = combine(a, b, r, sum0);
                    const uint64_t lo = (uint64_t)sum, hi = (uint64_t)(sum >> 64);
                    if (EDGE && !(mrow + dr < m_lim && n < p.N)) continue;
                    const long o = o0 + (long)dr * p.ldc;
                    // bits [sh, sh + 64): the upper word comes in through two shifts so that sh == 0 needs no case of its own
                    p.C[o] = (int64_t)((lo >> sh) | ((hi << 1) << (63 - sh)));
                    if (REM) p.R[o] = (int64_t)(lo & rmask);
                }
            }
    };
    const bool edge = m0 + BM > m_lim || n0 + BN > p.N;
    if (p.R) { if (edge) store_tile(std::true_type(), std::true_type()); else store_tile(std::false_type(), std::true_type()); }
    else { if (edge) store_tile(std::true_type(), std::false_type()); else store_tile(std::false_type(), std::false_type()); }
}

template <int NA, int NB, int WVM, int WVN, int WM, int WN, int KK, bool B32, bool BKM, bool APL, bool GRP = false, bool BRS = false, int DMAX = 16,
          bool BPL = false>
__global__ __launch_bounds__(64 * WVM * WVN) void gemm_mfma_kernel(MfmaParams p)
{
    gemm_mfma_block<NA, NB, WVM, WVN, WM, WN, KK, B32, BKM, APL, GRP, BRS, DMAX, BPL>(p, (int)blockIdx.x);
}

// The same product behind a guard word: nothing happens unless *p.guard is non-zero (the verdict of the speculative launch
// in front of it: its digit counts did not cover the operands), and then the grid, one workgroup per compute unit, walks
// the workgroup ids of an ordinary launch.  A guarded launch almost always finds nothing to do, and thousands of
// workgroups with 80 KB of LDS each would take tens of microseconds to find that out.
template <int NA, int NB, int WVM, int WVN, int WM, int WN, int KK, bool B32, int DMAX = 16>
__global__ __launch_bounds__(64 * WVM * WVN) void gemm_mfma_guarded_kernel(MfmaParams p)
{
    const unsigned long long verdict = __atomic_load_n(p.guard, __ATOMIC_RELAXED);            // (the same for every thread of the launch)
    if (verdict == 0) return;
    if (verdict == 1 && (NA > 5 || NB > 5)) {
        // five digits cover both operands (the fold kernel has seen every element): a third of the digit pairs of (9,9)
        constexpr int NA5 = NA > 5 ? 5 : NA, NB5 = NB > 5 ? 5 : NB;
        for (int block = (int)blockIdx.x; block < p.walk_blocks; block += (int)gridDim.x) {
            gemm_mfma_block<NA5, NB5, WVM, WVN, WM, WN, KK, B32, false, false, false, false, 16, false>(p, block);
            __syncthreads();
        }
        return;
    }
    for (int block = (int)blockIdx.x; block < p.walk_blocks; block += (int)gridDim.x) {
        gemm_mfma_block<NA, NB, WVM, WVN, WM, WN, KK, B32, false, false, false, false, DMAX, false>(p, block);
        __syncthreads();            // (the LDS stages and the range words in them are used again)
    }
}

// Adds the `split` partial sums of every tail tile, applies the rounding term and the shift, and stores C and R.
// Thread layout and element order are those of the GEMM kernel's epilogue.
// The last `fold.parts` workgroups fold the ranges (the GEMM kernel has left them by then), which saves a launch.
template <int WVM, int WVN, int WM, int WN>
__global__ __launch_bounds__(64 * WVM * WVN) void gemm_split_finish_kernel(MfmaParams p, FoldArgs fold)
{
    if (blockIdx.x >= gridDim.x - fold.parts) {
        range_fold_body(fold, (int)(blockIdx.x - (gridDim.x - fold.parts)));
        return;
    }
    constexpr int T = 64 * WVM * WVN, BM = 32 * WM * WVM, BN = 32 * WN * WVN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WVN, wn = wave % WVN;
    const int per_batch = p.tiles_m * p.tiles_n;
    const int tail_tile = blockIdx.x / p.finish_rq, rq = blockIdx.x % p.finish_rq, lin = p.main_tiles + tail_tile;
    const int r_per = 16 / p.finish_rq;
    const int g = lin / per_batch, rem = lin - g * per_batch;
    const int tn = p.n_fastest ? rem % p.tiles_n : rem / p.tiles_m, tm = p.n_fastest ? rem / p.tiles_n : rem - tn * p.tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;
    const uint64_t rmask = p.shift ? ((1ull << p.shift) - 1) : 0;
    const long qs = (long)(T / 64) * (WM * WN * 16);          // from one slice to the next
    // the registers of this workgroup's share, RPER at a time with all their slices' loads under way together (one
    // output at a time, a thread has `split` loads in flight and the launch lives on latency)
    auto finish = [&](auto rper_tag) {
        constexpr int RPER = decltype(rper_tag)::value;
#pragma unroll
        for (int a = 0; a < WM; a++)
#pragma unroll
            for (int b = 0; b < WN; b++) {
                const int n = n0 + (wn * WN + b) * 32 + (lane & 31);
                const int r0 = rq * RPER;
                const long q0 = ((long)tail_tile * p.split * (T / 64) + wave) * (WM * WN * 16) + (a * WN + b) * 16 + r0;
                uint64_t lo[RPER], hi[RPER];
                bool live[RPER];
#pragma unroll
                for (int r4 = 0; r4 < RPER; r4++) {
                    const int r = r0 + r4;
                    lo[r4] = (uint64_t)p.init;
                    hi[r4] = (uint64_t)(p.init >> 63);
                    live[r4] = m0 + (wm * WM + a) * 32 + 8 * (r >> 2) + (r & 3) < p.M;      // (uniform over the wave; the others were never written)
                }
                if (p.part64) {
                    uint64_t s[RPER];
#pragma unroll
                    for (int r4 = 0; r4 < RPER; r4++) s[r4] = 0;
#pragma unroll 4
                    for (int sidx = 0; sidx < p.split; sidx++)
#pragma unroll
                        for (int r4 = 0; r4 < RPER; r4++)
                            s[r4] += p.partials[(q0 + r4 + sidx * qs) * 64 + lane];      // (rows past M: slots nobody wrote, read and dropped)
#pragma unroll
                    for (int r4 = 0; r4 < RPER; r4++) {
                        const uint64_t t = lo[r4] + s[r4];
                        hi[r4] += (uint64_t)((int64_t)s[r4] >> 63) + (t < lo[r4] ? 1 : 0);
                        lo[r4] = t;
                    }
                } else {
#pragma unroll 2
                    for (int sidx = 0; sidx < p.split; sidx++)
#pragma unroll
                        for (int r4 = 0; r4 < RPER; r4++)
                        {
                            const uint64_t plo = p.partials[(q0 + r4 + sidx * qs) * 128 + lane];
                            const uint64_t phi = p.partials[(q0 + r4 + sidx * qs) * 128 + 64 + lane];
                            const uint64_t t = lo[r4] + plo;
                            hi[r4] += phi + (t < lo[r4] ? 1 : 0);
                            lo[r4] = t;
                        }
                }
#pragma unroll
                for (int r4 = 0; r4 < RPER; r4++) {
                    const int r = r0 + r4;
                    const int m = m0 + (wm * WM + a) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (live[r4] && m < p.M && n < p.N) {
                        const long o = (long)g * p.sC + (long)m * p.ldc + n;
                        p.C[o] = (int64_t)(p.shift == 0 ? lo[r4] : ((lo[r4] >> p.shift) | (hi[r4] << (64 - p.shift))));
                        if (p.R) p.R[o] = (int64_t)(lo[r4] & rmask);
                    }
                }
            }
    };
    if (r_per == 4) finish(std::integral_constant<int, 4>());
    else if (r_per == 2) finish(std::integral_constant<int, 2>());
    else finish(std::integral_constant<int, 1>());
}

// ---- kernel tables -------------------------------------------------------------------------------------
typedef void (*MfmaKernel)(MfmaParams);
typedef void (*FinishKernel)(MfmaParams, FoldArgs);
typedef void (*PlanesKernel)(MfmaParams, unsigned char *, int, int, unsigned long long *);

enum Variant { kB64Fly = 0, kB64Planes, kB32Fly, kB32Planes, kB64KmajorFly, kB32KmajorFly, kB64Group, kB32Group, kB64FlyRs, kB32FlyRs,
               kB64PlanesBoth, kB64FlyBPlanes, kB64GroupBPlanes, kVariants };     // the last three: B from prepared digit planes

struct Instance {
    int na, nb, bm, bn, threads, kk;
    bool skinny;                 // 32-row tiles for M <= 32
    int dmax;                    // diagonals from this one up are left out (16: none but the 2^128 one)
    MfmaKernel fn[kVariants];
    PlanesKernel planes[2];      // [b32]: the owned-k pattern follows the element size of B
    FinishKernel finish;         // adds up the partial sums of split tail tiles (and folds the ranges)
    MfmaKernel guarded[2];       // [b32]: the guarded form for row-major B, A split on the fly (the widest instances only)
};


// KKSEL: MFMA k-depths (of 32) per pipeline step.  B32ONLY: an instance for int32 B alone.  The 32-row kernels live on
// the bytes they keep in flight, and a step of int32 weights is half the bytes of a step of int64 weights: with two
// depths per step they stream as much per step as the int64 kernels do (where the two LDS stages still fit).
// BPLONLY: an instance for grouped launches on prepared planes of B alone (deeper steps for them: more bytes in flight).
template <int NA, int NB, bool SKINNY = false, int DMAX = 16, int KKSEL = ZK_KK(0), bool B32ONLY = false, bool BPLONLY = false>
static Instance make_instance()
{
    constexpr int DD = (NA + NB - 1) > DMAX ? DMAX : (NA + NB - 1);      // diagonals kept = accumulator sets
    static_assert(!SKINNY || DD <= 10, "skinny tiles keep two waves per SIMD");
    // narrow: 8 waves as 2x4, 64x32 per wave (128x128); mid: 8 waves as 4x2, 32x32 per wave (128x64);
    // wide: 4 waves as 2x2, 32x32 per wave (64x64, one wave per SIMD because of the accumulator count)
    // skinny (M <= 32): 8 waves as 1x8, 32x32 per wave (32x256)
    constexpr int WVM = SKINNY ? 1 : (DD <= 5 ? 2 : (DD <= 10 ? 4 : 2));
    constexpr int WVN = SKINNY ? 8 : (DD <= 5 ? 4 : 2);
    constexpr int WM = SKINNY ? 1 : (DD <= 5 ? 2 : 1), WN = 1;
    constexpr int KK = KKSEL;
    static_assert(!B32ONLY || NB <= 5, "int32 values never need more than five digits");
    Instance s;
    s.na = NA; s.nb = NB; s.bm = 32 * WM * WVM; s.bn = 32 * WN * WVN; s.threads = 64 * WVM * WVN; s.kk = KK;
    s.skinny = SKINNY;
    s.dmax = DMAX;
    for (int v = 0; v < kVariants; v++) s.fn[v] = nullptr;
    s.guarded[0] = s.guarded[1] = nullptr;
    // every operand fits nine digits, every int32 five: these instances can stand behind any speculative launch
    if constexpr (NA == 9 && !SKINNY && DMAX == 16 && !B32ONLY && !BPLONLY) {
        if constexpr (NB == 9) s.guarded[0] = gemm_mfma_guarded_kernel<NA, NB, WVM, WVN, WM, WN, KK, false, DMAX>;
        if constexpr (NB == 5) s.guarded[1] = gemm_mfma_guarded_kernel<NA, NB, WVM, WVN, WM, WN, KK, true, DMAX>;
    }
    if constexpr (BPLONLY) {
        static_assert(SKINNY && !B32ONLY, "grouped launches run on the 32-row tiles");
        s.fn[kB64GroupBPlanes] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, false, false, false, true, false, DMAX, true>;
        s.finish = gemm_split_finish_kernel<WVM, WVN, WM, WN>;
        s.planes[0] = a_planes_kernel<NA, 2, KK>;
        s.planes[1] = a_planes_kernel<NA, 4, KK>;
        return s;
    }
    if constexpr (!B32ONLY) {
        s.fn[kB64Fly] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, false, false, false, false, false, DMAX>;
        s.fn[kB64Planes] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, false, false, true, false, false, DMAX>;
        s.fn[kB64KmajorFly] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, false, true, false, false, false, DMAX>;
    }
    if constexpr (!B32ONLY && KK == 1 && !SKINNY)
        s.fn[kB64PlanesBoth] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, false, false, true, false, false, DMAX, true>;
    if constexpr (!B32ONLY && KK == 1 && SKINNY) {
        s.fn[kB64FlyBPlanes] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, false, false, false, false, false, DMAX, true>;
        s.fn[kB64GroupBPlanes] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, false, false, false, true, false, DMAX, true>;
    }
    if constexpr (NB <= 5) {          // int32 values never need more than five digits
        s.fn[kB32Fly] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, true, false, false, false, false, DMAX>;
        s.fn[kB32Planes] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, true, false, true, false, false, DMAX>;
        s.fn[kB32KmajorFly] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, true, true, false, false, false, DMAX>;
    }
    if constexpr (SKINNY) {          // grouped launches (one B per segment of rows) run on the 32-row tiles only
        if constexpr (!B32ONLY) s.fn[kB64Group] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, false, false, false, true, false, DMAX>;
        if constexpr (NB <= 5) s.fn[kB32Group] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, true, false, false, true, false, DMAX>;
        // and so do products whose B is divided by a power of two first (the model's head projection)
        if constexpr (!B32ONLY) s.fn[kB64FlyRs] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, false, false, false, false, true, DMAX>;
        if constexpr (NB <= 5) s.fn[kB32FlyRs] = gemm_mfma_kernel<NA, NB, WVM, WVN, WM, WN, KK, true, false, false, false, true, DMAX>;
    }
    s.finish = gemm_split_finish_kernel<WVM, WVN, WM, WN>;
    s.planes[0] = a_planes_kernel<NA, 2, KK>;
    s.planes[1] = a_planes_kernel<NA, 4, KK>;
    return s;
}

// the instance lists of the translation units
void mfma_instances_narrow(std::vector<Instance> &out);
void mfma_instances_mid(std::vector<Instance> &out);
void mfma_instances_wide(std::vector<Instance> &out);
void mfma_instances_pruned(std::vector<Instance> &out);
void mfma_instances_rows32(std::vector<Instance> &out);
void mfma_instances_rows32b(std::vector<Instance> &out);
void mfma_instances_rows32c(std::vector<Instance> &out);
void mfma_instances_rows32d(std::vector<Instance> &out);
void mfma_instances_rows32e(std::vector<Instance> &out);

}  // namespace zk
