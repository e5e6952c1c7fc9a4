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
#include <type_traits>

namespace zk {

typedef int v4i_g __attribute__((ext_vector_type(4)));
typedef long long v2l_g __attribute__((ext_vector_type(2)));

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
    // grouped matrix-vector launches: blockIdx.y is a row of A, whose B is that of the segment the row lies in
    const void *const *grp_b;                 // device array of `groups` device pointers
    const int *grp_seg;                       // device [groups + 1]: first row of every segment
    int groups;
    int chunk;                                // staged matrix-vector kernel: elements of A per staging round
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

// ---- one or two rows of A: a matrix-vector product -----------------------------------------------------------
// Decoding runs every projection, and the head always, on a single token (inference/model.py:1519, 1599-1606): the
// product is a stream over the weights with next to no reuse, and exact 128-bit multiply-adds on the vector ALU keep
// up with that stream, so nothing has to be guessed about the operands and one launch does it all.
// A wave takes one column of the output (a row of B); WPC waves share it, each taking every WPC-th stretch of K, and
// a workgroup of four waves covers 4 / WPC columns.  A lane loads 16 bytes of the B row at a time (two int64 or four
// int32 weights) and the matching elements of each A row, 4-8 such loads in flight, and keeps one 128-bit sum per
// output.  Bytes in flight are what this kernel lives on: with 8-byte loads of int32 weights it streamed 1.7 TB/s,
// with 16-byte loads 3.4 TB/s.
constexpr int kGemvMaxM = 2;
constexpr long kGemvTwoPassBytes = 64L << 20;

// A 128-bit sum kept as a 64-bit low word and a count of what went past it, so that adding a signed 64-bit product is
// four independent-looking instructions (sign word, add, add-with-carry twice) instead of a four-word carry chain.
struct SplitSum {
    uint64_t lo = 0;
    int32_t over = 0;                      // carries out of lo minus the negative addends: the sum is lo + 2^64 * over
    __device__ __forceinline__ void add(int64_t x)
    {
        const uint64_t t = lo + (uint64_t)x;
        over += (int32_t)(t < lo) + (int32_t)(x >> 63);
        lo = t;
    }
    __device__ __forceinline__ u128 total() const { return (u128)lo + ((u128)(i128)(int64_t)over << 64); }
};

template <bool B32, bool RESCALE, int MR, int WPC, bool GRP = false>
__global__ __launch_bounds__(256) void gemv_kernel(ValuParams p)
{
    // One column per wave: several columns per wave would share the loads of A, and measured slower at every size
    // (the head: 1.33 ms with four against 1.27 ms), so COLS stays a constant of the code rather than a choice.
    constexpr int COLS = 1;
    constexpr int UN = B32 ? 4 : 8;                    // 16-byte loads per B row in flight
    __shared__ u128 part[4][COLS][MR];
    typedef typename std::conditional<B32, int32_t, int64_t>::type BT;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int group = wave / WPC, slice = wave % WPC;
    const long n0 = ((long)blockIdx.x * (4 / WPC) + group) * COLS;
    const int g = blockIdx.y;
    const int64_t *Ag = p.A + (long)g * p.sA;
    const void *Bbase = p.B;
    if (GRP) {
        // the segment that holds row g: the last one that starts at or before it (empty segments share a start with
        // their successor and lose to it)
        int lo = 0, hi = p.groups - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (p.grp_seg[mid] <= g) lo = mid; else hi = mid - 1;
        }
        Bbase = p.grp_b[lo];
    }
    long brow[COLS];                                   // columns past N read the last row; their sums are dropped
#pragma unroll
    for (int c = 0; c < COLS; c++) brow[c] = (long)g * p.sB + (n0 + c < p.N ? n0 + c : p.N - 1) * p.ldbn;
    u128 acc[COLS][MR];
#pragma unroll
    for (int c = 0; c < COLS; c++)
#pragma unroll
        for (int m = 0; m < MR; m++) acc[c][m] = 0;

    // int32 weights without divisors: a = ah * 2^32 + al (ah signed, al unsigned) meets b in two 64-bit products, a
    // third of the multiplies of the general case, and each kind has its own split sum (weights 2^32 and 1)
    constexpr bool SPLIT = B32 && !RESCALE;
    SplitSum shi[SPLIT ? COLS : 1][SPLIT ? MR : 1], slo[SPLIT ? COLS : 1][SPLIT ? MR : 1];
    auto mac = [&](int c, int m, int64_t a, int64_t b) {
        if (SPLIT) {
            const int32_t b32 = (int32_t)b;
            shi[c][m].add((int64_t)(int32_t)(a >> 32) * (int64_t)b32);
            slo[c][m].add((int64_t)(uint64_t)(uint32_t)a * (int64_t)b32);            // |al * b| < 2^63
        } else {
            if (RESCALE) { a = rescale_operand(a, p.a_rs, p.a_shift); b = rescale_operand(b, p.b_rs, p.b_shift); }
            acc[c][m] += (u128)((i128)a * (i128)b);
        }
    };
    // units of EPL consecutive k (16 bytes of a B row): every pointer and stride keeps the 16-byte loads aligned
    // (decided on the host)
    constexpr int EPL = B32 ? 4 : 2;
    const int units = p.tiles_m ? p.K / EPL : 0;       // tiles_m doubles as the "vector loads allowed" flag here
    if (n0 < p.N) {
        for (int q0 = slice * 64 * UN; q0 < units; q0 += WPC * 64 * UN) {
            BT b[UN][COLS][EPL];
            int64_t a[UN][MR][EPL];
#pragma unroll
            for (int u = 0; u < UN; u++) {
                const int q = q0 + u * 64 + lane;
                const bool in = q < units;
#pragma unroll
                for (int c = 0; c < COLS; c++) {
#pragma unroll
                    for (int e = 0; e < EPL; e++) b[u][c][e] = 0;
                    if (in) {
                        if (B32) {
                            const v4i_g t = *(const ZK_GLOBAL_MEM v4i_g *)(reinterpret_cast<const int32_t *>(Bbase) + brow[c] + 4 * q);
                            b[u][c][0] = (BT)t[0]; b[u][c][1] = (BT)t[1]; b[u][c][2 % EPL] = (BT)t[2]; b[u][c][3 % EPL] = (BT)t[3];
                        } else {
                            const v2l_g t = *(const ZK_GLOBAL_MEM v2l_g *)(reinterpret_cast<const int64_t *>(Bbase) + brow[c] + 2 * q);
                            b[u][c][0] = (BT)t[0]; b[u][c][1] = (BT)t[1];
                        }
                    }
                }
#pragma unroll
                for (int m = 0; m < MR; m++)
#pragma unroll
                    for (int h = 0; h < EPL / 2; h++) {
                        a[u][m][2 * h] = a[u][m][2 * h + 1] = 0;
                        if (in) {
                            const longlong2 t = *reinterpret_cast<const longlong2 *>(Ag + (long)m * p.lda + (long)EPL * q + 2 * h);
                            a[u][m][2 * h] = t.x; a[u][m][2 * h + 1] = t.y;
                        }
                    }
            }
#pragma unroll
            for (int u = 0; u < UN; u++)
#pragma unroll
                for (int c = 0; c < COLS; c++)
#pragma unroll
                    for (int m = 0; m < MR; m++)
#pragma unroll
                        for (int e = 0; e < EPL; e++) mac(c, m, a[u][m][e], b[u][c][e]);
        }
        // what the units left over (all of K when vector loads are not allowed)
        for (int k = EPL * units + slice * 64 + lane; k < p.K; k += WPC * 64) {
#pragma unroll
            for (int c = 0; c < COLS; c++) {
                const int64_t bv = load_b<B32>(Bbase, brow[c] + k);
#pragma unroll
                for (int m = 0; m < MR; m++) mac(c, m, Ag[(long)m * p.lda + k], bv);
            }
        }
    }

    // lanes, then the waves of a group
#pragma unroll
    for (int c = 0; c < COLS; c++)
#pragma unroll
        for (int m = 0; m < MR; m++) {
            if (SPLIT) acc[c][m] = (shi[c][m].total() << 32) + slo[c][m].total();
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const uint64_t lo = (uint64_t)__shfl_xor((long long)(uint64_t)acc[c][m], off, 64);
                const uint64_t hi = (uint64_t)__shfl_xor((long long)(uint64_t)(acc[c][m] >> 64), off, 64);
                acc[c][m] += ((u128)hi << 64) | lo;
            }
        }
    if (WPC > 1) {
        if (lane == 0)
#pragma unroll
            for (int c = 0; c < COLS; c++)
#pragma unroll
                for (int m = 0; m < MR; m++) part[wave][c][m] = acc[c][m];
        __syncthreads();
        if (slice != 0) return;
#pragma unroll
        for (int c = 0; c < COLS; c++)
#pragma unroll
            for (int m = 0; m < MR; m++)
#pragma unroll
                for (int w = 1; w < WPC; w++) acc[c][m] += part[group * WPC + w][c][m];
    }
    if (lane != 0) return;
    const uint64_t rmask = p.shift ? ((1ull << p.shift) - 1) : 0;
#pragma unroll
    for (int c = 0; c < COLS; c++) {
        if (n0 + c >= p.N) break;
#pragma unroll
        for (int m = 0; m < MR; m++) {
            if (m >= p.M) break;
            const u128 sum = acc[c][m] + (u128)(i128)p.init;
            const long o = (long)g * p.sC + (long)m * p.ldc + n0 + c;
            p.C[o] = (int64_t)(uint64_t)((i128)sum >> p.shift);
            if (p.R) p.R[o] = (int64_t)((uint64_t)sum & rmask);
        }
    }
}

// One row of A against int32 weights with the row staged in LDS.  Every wave of a workgroup needs the whole row, and
// read from memory it costs twice the bytes of the weights it meets; staged once per workgroup it is split on the way in,
//     a = a2 * 2^42 + a1 * 2^21 + a0,   a0, a1 in [0, 2^21),   a2 in [-2^21, 2^21),
// so that a piece times an int32 weight stays below 2^52 in magnitude and a lane can add 1024 of them in a plain 64-bit
// accumulator: one v_mad_i64_i32 per piece, no carry bookkeeping, and the vector memory pipe carries weights only.
// The three sums of a column meet in 128 bits at the end.  K <= 65536 (1024 terms per lane), K % 4 == 0, 16-byte
// aligned rows of A and B (decided on the host).  A wave owns CPW consecutive columns.
constexpr int kStagedWaves = 8;
constexpr int kStagedLoads = 8;          // 16-byte loads of weights in flight per lane (shared out over the rows)
constexpr int kStagedChunk = 4096;       // elements of A per staging round (over all rows): 12 bytes of LDS each
constexpr int kStagedMaxK = 65536;

typedef int v4i_s __attribute__((ext_vector_type(4)));

template <int MR, int CPW, bool GRP>
__global__ __launch_bounds__(64 * kStagedWaves) void gemv32_staged_kernel(ValuParams p)
{
    constexpr int UN = kStagedLoads / MR, T = 64 * kStagedWaves;
    extern __shared__ __align__(16) int32_t staged[];          // [MR][3] planes of `chunk` elements
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = blockIdx.y;
    const int64_t *Ag = p.A + (long)g * p.sA;
    const int32_t *Bbase = reinterpret_cast<const int32_t *>(p.B) + (long)g * p.sB;
    if (GRP) {
        // the segment that holds row g: the last one that starts at or before it
        int lo = 0, hi = p.groups - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (p.grp_seg[mid] <= g) lo = mid; else hi = mid - 1;
        }
        Bbase = reinterpret_cast<const int32_t *>(p.grp_b[lo]);
    }
    const int chunk = p.chunk;
    const v4i_s *plane[MR][3];
#pragma unroll
    for (int m = 0; m < MR; m++)
#pragma unroll
        for (int i = 0; i < 3; i++) plane[m][i] = reinterpret_cast<const v4i_s *>(staged + (3 * m + i) * chunk);
    const long n_first = ((long)blockIdx.x * kStagedWaves + wave) * CPW;
    int64_t acc[MR][CPW][3];
#pragma unroll
    for (int m = 0; m < MR; m++)
#pragma unroll
        for (int c = 0; c < CPW; c++) acc[m][c][0] = acc[m][c][1] = acc[m][c][2] = 0;

    for (int k0 = 0; k0 < p.K; k0 += chunk) {
        const int len = p.K - k0 < chunk ? p.K - k0 : chunk;
        if (k0) __syncthreads();
#pragma unroll
        for (int m = 0; m < MR; m++) {
            int2 *s0 = reinterpret_cast<int2 *>(staged + (3 * m) * chunk), *s1 = reinterpret_cast<int2 *>(staged + (3 * m + 1) * chunk),
                 *s2 = reinterpret_cast<int2 *>(staged + (3 * m + 2) * chunk);
            for (int k = 2 * threadIdx.x; k < len; k += 2 * T) {
                const longlong2 t = *reinterpret_cast<const longlong2 *>(Ag + (long)m * p.lda + k0 + k);
                s0[k >> 1] = make_int2((int)((uint32_t)t.x & 0x1FFFFFu), (int)((uint32_t)t.y & 0x1FFFFFu));
                s1[k >> 1] = make_int2((int)((uint32_t)(t.x >> 21) & 0x1FFFFFu), (int)((uint32_t)(t.y >> 21) & 0x1FFFFFu));
                s2[k >> 1] = make_int2((int)(t.x >> 42), (int)(t.y >> 42));
            }
        }
        __syncthreads();
        const int units = len >> 2;
#pragma unroll
        for (int c = 0; c < CPW; c++) {
            const long n = n_first + c < p.N ? n_first + c : p.N - 1;      // columns past N read the last row; dropped below
            const ZK_GLOBAL_MEM v4i_s *brow = (const ZK_GLOBAL_MEM v4i_s *)(Bbase + n * p.ldbn + k0);
            for (int q0 = 0; q0 < units; q0 += 64 * UN) {
                v4i_s b[UN];
#pragma unroll
                for (int u = 0; u < UN; u++) {
                    const int q = q0 + u * 64 + lane;
                    b[u] = q < units ? __builtin_nontemporal_load(brow + q) : v4i_s{ 0, 0, 0, 0 };
                }
#pragma unroll
                for (int u = 0; u < UN; u++) {
                    int q = q0 + u * 64 + lane;
                    q = q < units ? q : units - 1;                           // (its weights are zero)
#pragma unroll
                    for (int m = 0; m < MR; m++)
#pragma unroll
                        for (int i = 0; i < 3; i++) {
                            const v4i_s x = plane[m][i][q];
                            acc[m][c][i] += (int64_t)x.x * b[u].x + (int64_t)x.y * b[u].y + (int64_t)x.z * b[u].z + (int64_t)x.w * b[u].w;
                        }
                }
            }
        }
    }

    const uint64_t rmask = p.shift ? ((1ull << p.shift) - 1) : 0;
#pragma unroll
    for (int m = 0; m < MR; m++)
#pragma unroll
        for (int c = 0; c < CPW; c++) {
            u128 sum = (u128)((i128)acc[m][c][0] + ((i128)acc[m][c][1] << 21) + ((i128)acc[m][c][2] << 42));
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const uint64_t lo = (uint64_t)__shfl_xor((long long)(uint64_t)sum, off, 64);
                const uint64_t hi = (uint64_t)__shfl_xor((long long)(uint64_t)(sum >> 64), off, 64);
                sum += ((u128)hi << 64) | lo;
            }
            if (lane == 0 && n_first + c < p.N) {
                sum += (u128)(i128)p.init;
                const long o = (long)g * p.sC + (long)m * p.ldc + n_first + c;
                p.C[o] = (int64_t)(uint64_t)((i128)sum >> p.shift);
                if (p.R) p.R[o] = (int64_t)((uint64_t)sum & rmask);
            }
        }
}

static int device_cus()
{
    static int cus = 0;
    if (!cus) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus = n;
    }
    return cus;
}

// Launches the staged kernel if the product is one it takes: one or two rows (per batch or segment row), int32 weights,
// no divisors, K a multiple of four up to kStagedMaxK, 16-byte aligned rows, and enough columns for a workgroup per
// compute unit (a narrower output is better served by waves that share a column along K).
template <bool GRP>
static bool gemv32_staged_launch(ValuParams p, long rows, int cus)
{
    if (p.K % 4 != 0 || p.K > kStagedMaxK || p.K < 256 || rows > 65535 || p.M < 1 || p.M > 2) return false;
    const long wg1 = ((p.N + kStagedWaves - 1) / kStagedWaves) * rows;
    if (wg1 < cus) return false;
    p.chunk = p.K < kStagedChunk / p.M ? p.K : kStagedChunk / p.M;      // 48 KB of LDS: three workgroups per compute unit
    const size_t lds = (size_t)3 * p.M * p.chunk * sizeof(int32_t);
    // more columns per wave (the staging is shared by more of them) while that leaves two workgroups per compute unit
    const long wg4 = ((p.N + 4 * kStagedWaves - 1) / (4 * kStagedWaves)) * rows;
    const long wg2 = ((p.N + 2 * kStagedWaves - 1) / (2 * kStagedWaves)) * rows;
    auto launch = [&](auto mr_tag, auto cpw_tag) {
        constexpr int MR = decltype(mr_tag)::value, CPW = decltype(cpw_tag)::value;
        static_assert(3 * kStagedChunk * sizeof(int32_t) <= 64 * 1024, "the staging planes fit the default dynamic LDS limit");
        auto fn = gemv32_staged_kernel<MR, CPW, GRP>;
        const dim3 grid((unsigned)((p.N + CPW * kStagedWaves - 1) / (CPW * kStagedWaves)), (unsigned)rows);
        fn<<<grid, dim3(64 * kStagedWaves), lds, 0>>>(p);
        return true;
    };
    typedef std::integral_constant<int, 1> I1;
    typedef std::integral_constant<int, 2> I2;
    typedef std::integral_constant<int, 4> I4;
    if (p.M == 2) return wg2 >= 2L * cus ? launch(I2(), I2()) : launch(I2(), I1());
    if (wg4 >= 2L * cus) return launch(I1(), I4());
    if (wg2 >= 2L * cus) return launch(I1(), I2());
    return launch(I1(), I1());
}

// The same for n-contiguous B (the per-head weights of `bshd,hdc->bshc`): a lane owns an output column and walks K, the
// loads of a row of B are contiguous over the wave, and the elements of A are the same for every lane.
template <bool B32, bool RESCALE, int MR>
__global__ __launch_bounds__(256) void gemv_kmajor_kernel(ValuParams p)
{
    const long n = (long)blockIdx.x * 256 + threadIdx.x;
    const int g = blockIdx.y;
    if (n >= p.N) return;
    const int64_t *Ag = p.A + (long)g * p.sA;
    const long b0 = (long)g * p.sB + n;
    u128 acc[MR];
#pragma unroll
    for (int m = 0; m < MR; m++) acc[m] = 0;
#pragma unroll 4
    for (int k = 0; k < p.K; k++) {
        int64_t b = load_b<B32>(p.B, b0 + (long)k * p.ldbk);
        if (RESCALE) b = rescale_operand(b, p.b_rs, p.b_shift);
#pragma unroll
        for (int m = 0; m < MR; m++) {
            int64_t a = Ag[(long)m * p.lda + k];
            if (RESCALE) a = rescale_operand(a, p.a_rs, p.a_shift);
            acc[m] += (u128)((i128)a * (i128)b);
        }
    }
    const uint64_t rmask = p.shift ? ((1ull << p.shift) - 1) : 0;
#pragma unroll
    for (int m = 0; m < MR; m++) {
        if (m >= p.M) break;
        const u128 sum = acc[m] + (u128)(i128)p.init;
        const long o = (long)g * p.sC + (long)m * p.ldc + n;
        p.C[o] = (int64_t)(uint64_t)((i128)sum >> p.shift);
        if (p.R) p.R[o] = (int64_t)((uint64_t)sum & rmask);
    }
}

template <bool B32, bool RESCALE, int MR>
static void gemv_launch3(const ValuParams &p, int G)
{
    // enough waves to keep the weight stream busy: four per column for a narrow output, one for a wide one
    const long waves1 = (long)p.N * G;
    if (waves1 >= 8192) gemv_kernel<B32, RESCALE, MR, 1><<<dim3((unsigned)((p.N + 3) / 4), (unsigned)G), dim3(256), 0, 0>>>(p);
    else if (waves1 >= 4096) gemv_kernel<B32, RESCALE, MR, 2><<<dim3((unsigned)((p.N + 1) / 2), (unsigned)G), dim3(256), 0, 0>>>(p);
    else gemv_kernel<B32, RESCALE, MR, 4><<<dim3((unsigned)p.N, (unsigned)G), dim3(256), 0, 0>>>(p);
}

bool gemm_gemv_grouped_launch(const GroupedDesc &d)
{
    if (d.rows < 1 || d.rows > 65535 || d.N < 1 || d.K < 1 || d.groups < 1) return false;
    ValuParams p = {};
    p.A = d.A; p.B = nullptr; p.C = d.C; p.R = d.R;
    p.lda = d.lda; p.sA = d.lda; p.ldbn = d.K; p.ldbk = 1; p.sB = 0; p.ldc = d.ldc; p.sC = d.ldc;
    p.M = 1; p.N = d.N; p.K = d.K; p.shift = d.shift;
    p.init = d.init; p.a_rs = 1; p.b_rs = 1; p.a_shift = 0; p.b_shift = 0;
    p.grp_b = d.B; p.grp_seg = d.seg; p.groups = d.groups;
    // 16-byte loads: rows of A by their pointer and stride; every expert's B is taken to start on a 16-byte boundary
    // (a tensor of its own), its rows follow from K
    const size_t esz = d.b32 ? 4 : 8;
    p.tiles_m = ((((uintptr_t)d.A | (uintptr_t)(d.lda * 8)) & 15) == 0 && ((size_t)d.K * esz) % 16 == 0) ? 1 : 0;
    if (d.b32 && p.tiles_m && gemv32_staged_launch<true>(p, d.rows, device_cus())) return true;
    if (d.rows > 32) return false;         // past that the 32-row MFMA kernels are as fast as the kernel below
    const long waves1 = (long)d.N * d.rows;
    const unsigned rows = (unsigned)d.rows;
#define ZK_GEMVG(B32) do {                                                                                                  \
        if (waves1 >= 8192) gemv_kernel<B32, false, 1, 1, true><<<dim3((unsigned)((d.N + 3) / 4), rows), dim3(256), 0, 0>>>(p);      \
        else if (waves1 >= 4096) gemv_kernel<B32, false, 1, 2, true><<<dim3((unsigned)((d.N + 1) / 2), rows), dim3(256), 0, 0>>>(p);  \
        else gemv_kernel<B32, false, 1, 4, true><<<dim3((unsigned)d.N, rows), dim3(256), 0, 0>>>(p);                                  \
    } while (0)
    if (d.b32) ZK_GEMVG(true); else ZK_GEMVG(false);
#undef ZK_GEMVG
    return true;
}

bool gemm_gemv_launch(const GemmDesc &d)
{
    // three or four rows: two passes of two rows while the matrix is small enough for the launch count to matter more
    // than a second pass over it (the MFMA route is four launches however small the product)
    if (d.M > kGemvMaxM && d.M <= 2 * kGemvMaxM && d.G >= 1 && d.N >= 1 && d.K >= 1 &&
        (long)d.G * d.N * d.K * (d.b32 ? 4 : 8) <= kGemvTwoPassBytes) {
        for (int m0 = 0; m0 < d.M; m0 += kGemvMaxM) {
            GemmDesc h = d;
            h.M = d.M - m0 < kGemvMaxM ? d.M - m0 : kGemvMaxM;
            h.A = d.A + (long)m0 * d.lda;
            h.C = d.C + (long)m0 * d.ldc;
            h.R = d.R ? d.R + (long)m0 * d.ldc : nullptr;
            if (!gemm_gemv_launch(h)) return false;        // (the checks below do not depend on the row count)
        }
        return true;
    }
    if (d.M < 1 || d.M > kGemvMaxM || d.G > 65535 || d.N < 1 || d.K < 1) return false;
    const bool kmajor = d.ldbn == 1 && d.ldbk != 1;
    if (!kmajor && d.ldbk != 1) return false;
    // an n-contiguous B is walked by one thread per column: fine for the short K of the einsum that has it, not for more
    if (kmajor && d.K > 1024) return false;
    ValuParams p = {};
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
    // the 16-byte loads need 16-byte aligned rows of A and of B
    const size_t esz = d.b32 ? 4 : 8;
    const bool a_ok = (((uintptr_t)d.A | (uintptr_t)(d.lda * 8) | (uintptr_t)(d.sA * 8)) & 15) == 0;
    const bool b_ok = (((uintptr_t)d.B | (uintptr_t)(d.ldbn * esz) | (uintptr_t)(d.sB * esz)) & 15) == 0;
    p.tiles_m = (a_ok && b_ok) ? 1 : 0;
    const bool rescale = d.a_rs != 1 || d.b_rs != 1;
    if (kmajor) {
        const dim3 grid((unsigned)((d.N + 255) / 256), (unsigned)d.G);
#define ZK_GEMVK(B32, RS) do { if (d.M == 1) gemv_kmajor_kernel<B32, RS, 1><<<grid, dim3(256), 0, 0>>>(p); \
                               else gemv_kmajor_kernel<B32, RS, 2><<<grid, dim3(256), 0, 0>>>(p); } while (0)
        if (d.b32) { if (rescale) ZK_GEMVK(true, true); else ZK_GEMVK(true, false); }
        else { if (rescale) ZK_GEMVK(false, true); else ZK_GEMVK(false, false); }
#undef ZK_GEMVK
        return true;
    }
    if (d.b32 && !rescale && p.tiles_m && gemv32_staged_launch<false>(p, d.G, device_cus())) return true;
#define ZK_GEMV(B32, RS) do { if (d.M == 1) gemv_launch3<B32, RS, 1>(p, d.G); else gemv_launch3<B32, RS, 2>(p, d.G); } while (0)
    if (d.b32) { if (rescale) ZK_GEMV(true, true); else ZK_GEMV(true, false); }
    else { if (rescale) ZK_GEMV(false, true); else ZK_GEMV(false, false); }
#undef ZK_GEMV
    return true;
}

}  // namespace zk
