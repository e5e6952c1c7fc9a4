// GEMM for a handful of rows (M <= 16 per row tile): weight streams on v_mfma_i32_16x16x64_i8, digit counts taken
// from the data.
//
// A product of a few activation rows with a wide weight matrix (the MLA down-projections on a short prompt, the routed
// experts of a MoE layer with ~8 tokens each) is bound by the one pass over the weights, and the 32-row tiles of the
// general kernel multiply mostly padding there.  This kernel uses the 16x16x64 i8 MFMA, whose operand fragment is 16
// bytes of ONE row per lane: lane (i, q) = (lane % 16, lane / 16) holds 16 of the 64 k of a step for row i.  A lane's
// fragment is therefore a few 16-byte pieces of its own row (the four lanes of a row read 64 contiguous bytes per
// load): the raw elements travel from global memory straight into LDS (global_load_lds_dwordx4, no registers held
// while they are under way), each lane reads back what it loaded, splits it into balanced base-256 digits in
// registers (see gemm_mfma.hip for the digit scheme) and feeds the matrix pipe.  Which k a fragment byte stands for
// does not matter as long as both operands agree, so the byte order follows the loads.
//
// Nothing is guessed.  Before a step is split, the wavefront ORs the magnitudes of what it loaded and picks the digit
// counts that step needs (3, 4 or 5 per operand, accumulated in nine int32 diagonals per tile).  A wavefront that
// meets values beyond five digits (2^38 and up: nothing a model produces) drops what it has and recomputes its
// outputs with 128-bit multiply-adds on the vector ALU.  Results are exact for every input, no range travels to the
// host, and the call never waits.
//
// A workgroup is four wavefronts on the same 16 rows and the same slice of K, each with its own group of columns.
// The rows of A are loaded once per workgroup (every wavefront a quarter) into a ring of four steps that all four read;
// each wavefront has a ring of three steps of its own weights.  What bounds such a stream is the bytes under way:
// the rings keep about 100 KB of weights per compute unit in flight, at the price of one barrier per step.
// With one slice of K a wavefront stores C and R itself.  With several (a launch too small to fill the device
// otherwise) every workgroup leaves its wavefronts' 128-bit sums in slots of scratch and a second, small launch adds
// the slots, applies rounding term and shift and stores.
#include "gemm_mfma_kernels.h"
#include "lds_dma.h"

#include <cstdlib>
#include <mutex>

namespace zk {

struct Rows16Params {
    const int64_t *A;
    const void *B;
    int64_t *C, *R;
    long lda, sA, ldb, sB, ldc, sC;      // element strides: A[g*sA + m*lda + k], B[g*sB + n*ldb + k]
    int G, M, N, K, shift, b_shift;
    int64_t init;
    int row_tiles, col_groups, nslices;
    unsigned long long *acc;             // split K: per (g, row tile, column group) and slice, the wavefront's 128-bit sums
    // grouped mode: rows of A and C form one segment per group, every group has its own B (see GroupedDesc)
    const int *grp_seg, *grp_tiles, *grp_ntiles;
    const void *const *grp_b;
    const unsigned long long *guard;     // when set: do nothing unless this word is non-zero
    unsigned items;                      // work items of the launch (the grid may be smaller: workgroups walk them)
};

constexpr int kR16Fast = 9;              // diagonals the accumulators hold: digit pairs up to (5, 5)
constexpr int kR16FoldSteps = 16;        // steps between folds of the accumulators (5 pairs * 64 * 2^14 * 16 < 2^31)
constexpr int kR16Waves = 4;             // wavefronts per workgroup (one per SIMD: the kernel takes most of the register file)
constexpr int kR16StagesA = 4;           // steps of A the workgroup's shared ring holds (8 KB each)
constexpr int kR16StagesW = 3;           // steps of weights a wavefront's own ring holds (8 KB each)

// 16-column tiles per wavefront: a step of a wavefront's weights is 8 KB either way
template <bool B32> struct R16Shape {
    static constexpr int kColTiles = B32 ? 2 : 1;
    static constexpr int kCols = 16 * kColTiles;
    static constexpr int kLoadsPerTile = B32 ? 4 : 8;                       // 16-byte loads per lane and column tile
    static_assert(kColTiles * kLoadsPerTile == 8, "eight loads of weights per lane and step");
};
constexpr int kR16LdsBytes = kR16StagesA * 8192 + kR16Waves * kR16StagesW * 8192;

// The 64 k of a step are dealt to (lane quarter q, fragment byte b) so that every load is 16 bytes and the four lanes
// of a row read 64 contiguous bytes:
//   int64 weights: byte b <-> k = 8*(b/2) + 2*q + b%2      (A and B: eight loads of two elements)
//   int32 weights: byte b <-> k = 16*(b/4) + 4*q + b%4     (B: four loads of four elements; A: eight loads of two)
template <bool B32>
__device__ __forceinline__ int frag_k(int q, int b) { return B32 ? 16 * (b >> 2) + 4 * q + (b & 3) : 8 * (b >> 1) + 2 * q + (b & 1); }

// sums[r] += sum_d acc[d][r] * 2^(8 d): diagonals in groups of four (a group stays below 2^57), the groups meet in 128 bits
template <int D>
__device__ __forceinline__ void fold_diagonals(const v4i (&acc)[D], u128 (&sums)[4])
{
#pragma unroll
    for (int r = 0; r < 4; r++) {
#pragma unroll
        for (int gq = 0; gq < (D + 3) / 4; gq++) {
            uint64_t s = (uint64_t)(int64_t)acc[4 * gq][r];
#pragma unroll
            for (int j = 1; j < 4; j++)
                if (4 * gq + j < D) s += (uint64_t)(int64_t)acc[4 * gq + j][r] << (8 * j);
            sums[r] += (u128)(i128)(int64_t)s << (32 * gq);
        }
    }
}

// One operand fragment as loaded: 16 elements of 64 bits (A, int64 weights) or of 32 bits (int32 weights), as the
// 16-byte pieces the loads delivered.
template <bool W32> struct RawFrag { v4i v[W32 ? 4 : 8]; };

template <bool W32>
__device__ __forceinline__ uint64_t magnitude_or(const RawFrag<W32> &f)
{
    // OR of x for x >= 0 and ~x otherwise: below 2^(8n-2) means n digits hold every element
    if (W32) {
        uint32_t m = 0;
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int z = 0; z < 4; z++) m |= (uint32_t)(f.v[j][z] ^ (f.v[j][z] >> 31));
        return m;
    }
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int s = f.v[j][2 * h + 1] >> 31;
            lo |= (uint32_t)(f.v[j][2 * h] ^ s);
            hi |= (uint32_t)(f.v[j][2 * h + 1] ^ s);
        }
    return ((uint64_t)hi << 32) | lo;
}

// digits (3, 4, 5, or 9 for "more") that hold every element of the wavefront whose magnitudes OR to m in some lane
__device__ __forceinline__ int wave_digits(uint64_t m)
{
    if (__builtin_amdgcn_ballot_w64(m >> 22 != 0) == 0) return 3;
    if (__builtin_amdgcn_ballot_w64(m >> 30 != 0) == 0) return 4;
    if (__builtin_amdgcn_ballot_w64(m >> 38 != 0) == 0) return 5;
    return 9;
}

template <int N, bool W32>
__device__ __forceinline__ void split_frag(const RawFrag<W32> &f, v4i (&out)[N])
{
    if (W32) {
        int x[16];
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int z = 0; z < 4; z++) x[4 * j + z] = f.v[j][z];
        split16_w32<N>(x, out);
    } else if (N <= 4) {
        int x[16];                  // values below 2^(8N-2): the low words say it all
#pragma unroll
        for (int j = 0; j < 8; j++) { x[2 * j] = f.v[j][0]; x[2 * j + 1] = f.v[j][2]; }
        split16_w32<N>(x, out);
    } else {
        int64_t x[16];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            x[2 * j] = (int64_t)(((uint64_t)(uint32_t)f.v[j][1] << 32) | (uint32_t)f.v[j][0]);
            x[2 * j + 1] = (int64_t)(((uint64_t)(uint32_t)f.v[j][3] << 32) | (uint32_t)f.v[j][2]);
        }
        split16<N>(x, out);
    }
}

template <int NA, int NB, bool B32>
__device__ __forceinline__ void step_fast(const RawFrag<false> &fa_raw, const RawFrag<B32> (&fw_raw)[R16Shape<B32>::kColTiles],
                                          v4i (&acc)[R16Shape<B32>::kColTiles][kR16Fast])
{
    v4i fa[NA];
    split_frag<NA, false>(fa_raw, fa);
#pragma unroll
    for (int ct = 0; ct < R16Shape<B32>::kColTiles; ct++) {
        v4i fb[NB];
        split_frag<NB, B32>(fw_raw[ct], fb);
#pragma unroll
        for (int i = 0; i < NA; i++)
#pragma unroll
            for (int j = 0; j < NB; j++)
                acc[ct][i + j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[i], fb[j], acc[ct][i + j], 0, 0, 0);
    }
}

template <bool B32, bool GRP>
__device__ __forceinline__ void rows16_item(const Rows16Params &p, unsigned item)
{
    typedef R16Shape<B32> S;
    constexpr int CT = S::kColTiles, LPT = S::kLoadsPerTile;
    constexpr int LPS = 2 + 8;                       // loads per lane and step: a quarter of A's eight, the weights' eight
    extern __shared__ __attribute__((aligned(16))) unsigned char r16_smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, li = lane & 15, q = lane >> 4;
    unsigned char *ring_a = r16_smem;                                               // [stage][load][lane] 16 bytes
    unsigned char *ring_w = r16_smem + kR16StagesA * 8192 + wave * (kR16StagesW * 8192);
    const unsigned ring_a_lds = (unsigned)(uintptr_t)ring_a, ring_w_lds = (unsigned)(uintptr_t)ring_w;   // LDS byte addresses

    // workgroup -> (batch or 32-row tile half, four column groups, K slice); the wavefronts take the column groups
    const int cg4 = (p.col_groups + kR16Waves - 1) / kR16Waves;
    int slice = 0;
    if (p.nslices > 1) { slice = (int)(item % (unsigned)p.nslices); item /= (unsigned)p.nslices; }
    const int cg = (int)(item % (unsigned)cg4) * kR16Waves + wave;
    item /= (unsigned)cg4;
    int g = 0, m0 = 0, m_lim = p.M;
    const void *b_base = p.B;
    long tile_id = 0;                       // index of (g, row tile, column group) among the launch's output tiles
    if (GRP) {
        // item = (32-row tile of the dispatch table, half): 16 rows each
        const int mt = (int)(item >> 1), half = (int)(item & 1);
        if (mt >= *p.grp_ntiles) return;                            // (the same for the whole workgroup)
        const int e = p.grp_tiles[2 * mt];
        m0 = p.grp_tiles[2 * mt + 1] + 16 * half;
        m_lim = p.grp_seg[e + 1];
        if (m0 >= m_lim) return;
        b_base = p.grp_b[e];
    } else {
        const int rt = (int)(item % (unsigned)p.row_tiles);
        g = (int)(item / (unsigned)p.row_tiles);
        m0 = rt * 16;
        tile_id = ((long)g * p.row_tiles + rt) * p.col_groups + cg;
    }
    // a wavefront past the last column group still loads its quarter of A and meets the others at the barriers
    const bool live = cg < p.col_groups;
    const int n0 = (live ? cg : 0) * S::kCols;

    // this lane's rows (clamped: the products of rows past the end land in outputs that are never stored)
    int am = m0 + li;
    am = am < m_lim ? am : m_lim - 1;
    const int64_t *a_row = p.A + (long)g * p.sA + (long)am * p.lda;
    const char *w_row[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ct++) {
        int n = n0 + 16 * ct + li;
        n = n < p.N ? n : p.N - 1;
        w_row[ct] = reinterpret_cast<const char *>(b_base) + ((long)g * p.sB + (long)n * p.ldb) * (B32 ? 4 : 8);
    }
    const bool vec = (((uintptr_t)p.A | (uintptr_t)(p.lda * 8) | (uintptr_t)(p.sA * 8)) & 15) == 0 &&
                     (((uintptr_t)b_base | (uintptr_t)(p.ldb * (B32 ? 4 : 8)) | (uintptr_t)(p.sB * (B32 ? 4 : 8))) & 15) == 0;

    const int ksteps = (p.K + 63) / 64;
    const int ks_begin = (int)((long)slice * ksteps / p.nslices), ks_end = (int)((long)(slice + 1) * ksteps / p.nslices);
    // steps that travel through the rings: whole ones, on 16-byte aligned rows; the others are loaded element by element
    const int full_end = vec ? (p.K / 64 < ks_end ? p.K / 64 : ks_end) : ks_begin;

    v4i acc[CT][kR16Fast];
    u128 sums[CT][4];
#pragma unroll
    for (int ct = 0; ct < CT; ct++) {
#pragma unroll
        for (int d = 0; d < kR16Fast; d++) acc[ct][d] = v4i{ 0, 0, 0, 0 };
#pragma unroll
        for (int r = 0; r < 4; r++) sums[ct][r] = 0;
    }
    auto fold = [&]() {
#pragma unroll
        for (int ct = 0; ct < CT; ct++) {
            fold_diagonals<kR16Fast>(acc[ct], sums[ct]);
#pragma unroll
            for (int d = 0; d < kR16Fast; d++) acc[ct][d] = v4i{ 0, 0, 0, 0 };
        }
    };

    // step ks on its way: this wavefront's quarter of A's eight pieces into the shared ring, its weights into its own
    auto issue = [&](int ks) {
        const int k0 = ks * 64;
        const unsigned base_a = ring_a_lds + ((ks - ks_begin) % kR16StagesA) * 8192;
        const unsigned base_w = ring_w_lds + ((ks - ks_begin) % kR16StagesW) * 8192;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            // (the piece number depends on the wavefront: every j is compiled, one is taken)
#pragma unroll
            for (int j = 0; j < 8; j++)
                if (j == 2 * wave + h) lds_dma16(a_row + k0 + frag_k<B32>(q, 2 * j), base_a + j * 1024);
        }
#pragma unroll
        for (int ct = 0; ct < CT; ct++)
#pragma unroll
            for (int j = 0; j < LPT; j++)
                lds_dma16(w_row[ct] + (long)(k0 + frag_k<B32>(q, (16 / LPT) * j)) * (B32 ? 4 : 8), base_w + (ct * LPT + j) * 1024);
    };

    RawFrag<false> fa;
    RawFrag<B32> fw[CT];
    int since_fold = 0;
    bool wide = false;
    // one step on the fragments in fa / fw: digit counts from the data, split, multiply
    auto process = [&]() {
        if (p.b_shift) {
            // weights divided by a power of two first (truncating toward zero)
#pragma unroll
            for (int ct = 0; ct < CT; ct++) {
                if (B32) {
#pragma unroll
                    for (int j = 0; j < LPT; j++)
#pragma unroll
                        for (int z = 0; z < 4; z++) fw[ct].v[j][z] = (int)tdiv_pow2((int64_t)fw[ct].v[j][z], p.b_shift > 31 ? 31 : p.b_shift);
                } else {
#pragma unroll
                    for (int j = 0; j < LPT; j++)
#pragma unroll
                        for (int h = 0; h < 2; h++) {
                            const int64_t x = (int64_t)(((uint64_t)(uint32_t)fw[ct].v[j][2 * h + 1] << 32) | (uint32_t)fw[ct].v[j][2 * h]);
                            const int64_t y = tdiv_pow2(x, p.b_shift);
                            fw[ct].v[j][2 * h] = (int)(uint32_t)y;
                            fw[ct].v[j][2 * h + 1] = (int)(uint32_t)((uint64_t)y >> 32);
                        }
                }
            }
        }
        uint64_t mw = 0;
#pragma unroll
        for (int ct = 0; ct < CT; ct++) mw |= magnitude_or<B32>(fw[ct]);
        const int na = wave_digits(magnitude_or<false>(fa));
        int nb = wave_digits(mw);
        if (B32 && nb > 5) nb = 5;                          // (an int32 never needs more)
        if (na > 5 || nb > 5) { wide = true; return; }
        switch ((na - 3) * 3 + (nb - 3)) {
        case 0: step_fast<3, 3, B32>(fa, fw, acc); break;
        case 1: step_fast<3, 4, B32>(fa, fw, acc); break;
        case 2: step_fast<3, 5, B32>(fa, fw, acc); break;
        case 3: step_fast<4, 3, B32>(fa, fw, acc); break;
        case 4: step_fast<4, 4, B32>(fa, fw, acc); break;
        case 5: step_fast<4, 5, B32>(fa, fw, acc); break;
        case 6: step_fast<5, 3, B32>(fa, fw, acc); break;
        case 7: step_fast<5, 4, B32>(fa, fw, acc); break;
        default: step_fast<5, 5, B32>(fa, fw, acc); break;
        }
        if (++since_fold == kR16FoldSteps) { fold(); since_fold = 0; }
    };

    // Three steps under way.  In iteration ks: this wavefront's loads of step ks have landed (at most the two steps issued
    // after it are outstanding); behind the barrier so have everybody's quarters of A, and everybody has read the step
    // before out of the ring; the step moves into registers; step ks + 3 is issued into the stages that just became free
    // (its weights into the stage read a moment ago, its rows of A into the stage of step ks - 1).
#pragma unroll
    for (int d = 0; d < kR16StagesW; d++)
        if (ks_begin + d < full_end) issue(ks_begin + d);
    for (int ks = ks_begin; ks < full_end; ks++) {
        const int behind = full_end - 1 - ks;
        if (behind >= 2) wait_vmcnt<2 * LPS>();
        else if (behind == 1) wait_vmcnt<LPS>();
        else wait_vmcnt<0>();
        __syncthreads();
        const unsigned char *src_a = ring_a + ((ks - ks_begin) % kR16StagesA) * 8192 + lane * 16;
        const unsigned char *src_w = ring_w + ((ks - ks_begin) % kR16StagesW) * 8192 + lane * 16;
#pragma unroll
        for (int j = 0; j < 8; j++) fa.v[j] = *reinterpret_cast<const v4i *>(src_a + j * 1024);
#pragma unroll
        for (int ct = 0; ct < CT; ct++)
#pragma unroll
            for (int j = 0; j < LPT; j++) fw[ct].v[j] = *reinterpret_cast<const v4i *>(src_w + (ct * LPT + j) * 1024);
        if (ks + kR16StagesW < full_end) {
            // (the reads above must have returned before their stage is overwritten)
            __builtin_amdgcn_s_waitcnt(0xC07F);            // lgkmcnt(0)
            issue(ks + kR16StagesW);
        }
        if (live && !wide) process();
    }
    wait_vmcnt<0>();
    // steps outside the rings (a partial last step, rows that are not 16-byte aligned): element by element
    for (int ks = full_end; ks < ks_end && live && !wide; ks++) {
        const int k0 = ks * 64, k_left = p.K - k0;
#pragma unroll
        for (int b = 0; b < 16; b++) {
            const int k = frag_k<B32>(q, b);
            const int64_t x = k < k_left ? a_row[k0 + k] : 0;
            fa.v[b >> 1][2 * (b & 1)] = (int)(uint32_t)x;
            fa.v[b >> 1][2 * (b & 1) + 1] = (int)(uint32_t)((uint64_t)x >> 32);
        }
#pragma unroll
        for (int ct = 0; ct < CT; ct++)
#pragma unroll
            for (int b = 0; b < 16; b++) {
                const int k = frag_k<B32>(q, b);
                if (B32) {
                    fw[ct].v[b >> 2][b & 3] = k < k_left ? reinterpret_cast<const int32_t *>(w_row[ct])[k0 + k] : 0;
                } else {
                    const int64_t x = k < k_left ? reinterpret_cast<const int64_t *>(w_row[ct])[k0 + k] : 0;
                    fw[ct].v[b >> 1][2 * (b & 1)] = (int)(uint32_t)x;
                    fw[ct].v[b >> 1][2 * (b & 1) + 1] = (int)(uint32_t)((uint64_t)x >> 32);
                }
            }
        process();
    }
    if (!live) return;
    fold();
    if (wide) {
        // Values beyond five digits (2^38) somewhere in this item's slice: every lane recomputes its outputs with
        // 128-bit multiply-adds on the vector ALU, straight from memory.  Slow and exact; model data never comes here.
#pragma unroll 1
        for (int o = 0; o < CT * 4; o++) {
            const int ct = o >> 2, r = o & 3;
            int m = m0 + 4 * q + r, n = n0 + 16 * ct + li;
            m = m < m_lim ? m : m_lim - 1;
            n = n < p.N ? n : p.N - 1;
            const int64_t *ar = p.A + (long)g * p.sA + (long)m * p.lda;
            const char *wr = reinterpret_cast<const char *>(b_base) + ((long)g * p.sB + (long)n * p.ldb) * (B32 ? 4 : 8);
            const int k_end = ks_end * 64 < p.K ? ks_end * 64 : p.K;
            u128 s = 0;
            for (int k = ks_begin * 64; k < k_end; k++) {
                int64_t w = B32 ? (int64_t)reinterpret_cast<const int32_t *>(wr)[k] : reinterpret_cast<const int64_t *>(wr)[k];
                if (p.b_shift) w = tdiv_pow2(w, p.b_shift);
                s += (u128)((i128)ar[k] * (i128)w);
            }
            // (static register indices: the sums stay in registers)
#pragma unroll
            for (int c2 = 0; c2 < CT; c2++)
#pragma unroll
                for (int r2 = 0; r2 < 4; r2++)
                    if (c2 == ct && r2 == r) sums[c2][r2] = s;
        }
    }

    if (p.nslices == 1) {
        // accumulator register r of lane (li, q) holds row 4*q + r, column li of its 16x16 tile
        const uint64_t rmask = p.shift ? ((1ull << p.shift) - 1) : 0;
#pragma unroll
        for (int ct = 0; ct < CT; ct++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int m = m0 + 4 * q + r, n = n0 + 16 * ct + li;
                if (m >= m_lim || n >= p.N) continue;
                const u128 s = sums[ct][r] + (u128)(i128)p.init;
                const uint64_t lo = (uint64_t)s, hi = (uint64_t)(s >> 64);
                const long o = (long)g * p.sC + (long)m * p.ldc + n;
                p.C[o] = (int64_t)((lo >> p.shift) | ((hi << 1) << (63 - p.shift)));
                if (p.R) p.R[o] = (int64_t)(lo & rmask);
            }
        return;
    }
    // Several slices: the sums go to this slice's slot of the tile's scratch, and a second launch adds the slots up.
    // (Finishing inside this kernel was measured first.  Adding into one slot with atomics: fourteen workgroups adding 512
    // sums each spent 3.4 us in dependent round trips to the memory side, and every further slice 0.3 us.  A ticket with
    // the last arriver adding the slots: a round trip for the stores, one for the ticket, and several for the loads,
    // since nothing that crosses the dies may be fenced or cached.  A launch boundary costs less than either.)
    u128 *slot = reinterpret_cast<u128 *>(p.acc) + ((long)tile_id * p.nslices + slice) * (CT * 4 * 64);
#pragma unroll
    for (int ct = 0; ct < CT; ct++)
#pragma unroll
        for (int r = 0; r < 4; r++) slot[(ct * 4 + r) * 64 + lane] = sums[ct][r];
}

// One workgroup per item (a tile of 16 rows, four column groups, a slice of K), or, behind a guard word, a grid of one
// workgroup per compute unit that walks the items: such a launch is the fallback behind a speculative launch of the
// 32-row kernels and almost always has nothing to do, which a grid of ten thousand workgroups of 128 KB of LDS each
// takes 60 us to find out.
template <bool B32, bool GRP>
__global__ __launch_bounds__(64 * kR16Waves) void gemm_rows16_kernel(Rows16Params p)
{
    if (p.guard && *p.guard == 0) return;            // (the same for every thread of the launch)
    for (unsigned item = blockIdx.x; item < p.items; item += gridDim.x) {
        rows16_item<B32, GRP>(p, item);
        if (item + gridDim.x < p.items) __syncthreads();           // (the rings are used again)
    }
}

// Adds the slots of every output tile, applies rounding term and shift, stores C and R.  Four threads share an output
// (each adds every fourth slice with all its loads under way at once, then the four meet through shuffles): the launch
// is a chain of one load latency, not of one per slice.
template <bool B32>
__global__ __launch_bounds__(256) void gemm_rows16_finish_kernel(Rows16Params p)
{
    constexpr int CT = R16Shape<B32>::kColTiles, PER = CT * 4 * 64;         // sums per slot
    const long idx = ((long)blockIdx.x * 256 + threadIdx.x) >> 2;
    const int part = threadIdx.x & 3;
    const long tile_id = idx / PER;
    const int o = (int)(idx - tile_id * PER), lane = o & 63, cr = o >> 6, ct = cr >> 2, r = cr & 3;
    const long tiles = (long)p.G * p.row_tiles * p.col_groups;
    if (tile_id >= tiles) return;                                          // (whole groups of four leave together)
    const int cg = (int)(tile_id % p.col_groups);
    const long t2 = tile_id / p.col_groups;
    const int rt = (int)(t2 % p.row_tiles), g = (int)(t2 / p.row_tiles);
    const int m = rt * 16 + 4 * (lane >> 4) + r, n = cg * R16Shape<B32>::kCols + 16 * ct + (lane & 15);
    const int groups = p.nslices;
    const u128 *slot = reinterpret_cast<const u128 *>(p.acc) + tile_id * groups * PER + o;
    u128 s = 0;
    for (int g0 = part; g0 < groups; g0 += 32) {
        u128 t[8];
#pragma unroll
        for (int j = 0; j < 8; j++) t[j] = g0 + 4 * j < groups ? slot[(long)(g0 + 4 * j) * PER] : (u128)0;
#pragma unroll
        for (int j = 0; j < 8; j++) s += t[j];
    }
    uint64_t lo = (uint64_t)s, hi = (uint64_t)(s >> 64);
#pragma unroll
    for (int off = 1; off < 4; off <<= 1) {
        const uint64_t olo = (uint64_t)__shfl_xor((long long)lo, off, 64), ohi = (uint64_t)__shfl_xor((long long)hi, off, 64);
        const uint64_t tlo = lo + olo;
        hi += ohi + (tlo < lo ? 1 : 0);
        lo = tlo;
    }
    if (part != 0 || m >= p.M || n >= p.N) return;
    const uint64_t ilo = (uint64_t)p.init, ihi = (uint64_t)(p.init >> 63);
    const uint64_t flo = lo + ilo;
    hi += ihi + (flo < lo ? 1 : 0);
    lo = flo;
    const long at = (long)g * p.sC + (long)m * p.ldc + n;
    p.C[at] = (int64_t)((lo >> p.shift) | ((hi << 1) << (63 - p.shift)));
    if (p.R) p.R[at] = (int64_t)(p.shift ? lo & ((1ull << p.shift) - 1) : 0);
}

}  // namespace zk

namespace zk {

// ---- host side ---------------------------------------------------------------------------------------------
// Scratch of the split-K launches, kept between calls: slots of 8 KB (the 128-bit sums of one wavefront: one output tile,
// one slice of K).  Every slot a launch reads has been written by that launch: nothing needs clearing.
static unsigned long long *g_r16_acc = nullptr;
static size_t g_r16_slots = 0;
static int g_r16_cus = 0;
static std::mutex g_r16_mu;              // host threads take turns in the launchers below (the scratch may be regrown, the attribute list filled)

constexpr size_t kR16SlotBytes = 8 * 64 * 16;
constexpr int kNoAllocMaxRows = 16;                        // limits of int64_bmm_broadcast_noalloc
constexpr long kNoAllocMaxOutputs = 1L << 20;

static void r16_release_locked()
{
    if (g_r16_acc) (void)hipFree(g_r16_acc);
    g_r16_acc = nullptr;
    g_r16_slots = 0;
}

size_t gemm_rows16_workspace_bytes()
{
    std::lock_guard<std::mutex> lock(g_r16_mu);
    return g_r16_slots * kR16SlotBytes;
}

void gemm_rows16_release_workspace()
{
    std::lock_guard<std::mutex> lock(g_r16_mu);
    r16_release_locked();
}

static int r16_cus()
{
    if (!g_r16_cus) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        g_r16_cus = n;
    }
    return g_r16_cus;
}

// 0: the buffer holds `slots` slots, 1: no memory (the caller runs without split K), -1: error recorded
static int r16_scratch(size_t slots)
{
    if (slots <= g_r16_slots) return 0;
    // the old buffer may still be in use by launches under way: the stream is drained first (this happens a few times
    // in a process, while the largest launch is still growing)
    if (g_r16_slots && hipStreamSynchronize(0) != hipSuccess) { set_error(kLaunchFailure, "gemm: cannot wait for the stream"); return -1; }
    r16_release_locked();
    if (hipMalloc(&g_r16_acc, slots * kR16SlotBytes) != hipSuccess) {
        (void)hipGetLastError();
        g_r16_acc = nullptr;
        return 1;
    }
    g_r16_slots = slots;
    return 0;
}

// How many slices of K.  One workgroup fits a compute unit, so a launch runs in rounds of `cus` workgroups; the count
// that minimises rounds x steps per wavefront wins, a split being charged the second launch.
static int r16_slices(long wg_tiles, int K, int cus)
{
    const int ksteps = (K + 63) / 64;
    // in units of one step of one wavefront (about a microsecond): start-up of a round, the finishing launch
    const double round_cost = 3.0, finish_cost = 4.0;
    int best = 1;
    double best_cost = 0;
    for (int n = 1; n == 1 || n <= ksteps / 2; n++) {
        const long rounds = (wg_tiles * n + cus - 1) / cus;
        const double cost = rounds * ((double)((ksteps + n - 1) / n) + round_cost) + (n > 1 ? finish_cost : 0.0);
        if (n == 1 || cost < best_cost) { best = n; best_cost = cost; }
    }
    return best;
}

static bool r16_fill(const GemmDesc &d, Rows16Params &p)
{
    if (d.a_rs != 1 || d.ldbk != 1 || d.M < 1 || d.M > 16 || d.N < 1 || d.K < 0 || d.G < 1) return false;
    int b_shift = 0;
    if (d.b_rs != 1) {
        if (d.b_rs <= 0 || (d.b_rs & (d.b_rs - 1)) != 0) return false;
        while (((int64_t)1 << b_shift) < d.b_rs) b_shift++;
    }
    const int cols = d.b32 ? R16Shape<true>::kCols : R16Shape<false>::kCols;
    p = Rows16Params{};
    p.A = d.A; p.B = d.B; p.C = d.C; p.R = d.R;
    p.lda = d.lda; p.sA = d.sA; p.ldb = d.ldbn; p.sB = d.sB; p.ldc = d.ldc; p.sC = d.sC;
    p.G = d.G; p.M = d.M; p.N = d.N; p.K = d.K; p.shift = d.shift; p.b_shift = b_shift; p.init = d.init;
    p.row_tiles = (d.M + 15) / 16;
    p.col_groups = (d.N + cols - 1) / cols;
    p.nslices = 1;
    return true;
}

typedef void (*Rows16Kernel)(Rows16Params);

static int r16_run(Rows16Kernel fn, const Rows16Params &params, long blocks)
{
    if (blocks > 0x7FFFFFF0L) return 1;
    constexpr int lds = kR16LdsBytes;
    Rows16Params p = params;
    p.items = (unsigned)blocks;
    if (p.guard && blocks > r16_cus()) blocks = r16_cus();
    static const void *raised[4] = {};
    bool seen = false;
    for (const void *f : raised) seen = seen || f == (const void *)fn;
    if (!seen) {
        if (hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) {
            set_error(kLaunchFailure, "gemm: cannot raise the LDS limit of the 16-row kernel to %d bytes", lds);
            return -1;
        }
        for (const void *&f : raised)
            if (!f) { f = (const void *)fn; break; }
    }
    fn<<<dim3((unsigned)blocks), dim3(64 * kR16Waves), lds, 0>>>(p);
    if (hipGetLastError() != hipSuccess) { set_error(kLaunchFailure, "gemm: the 16-row kernel could not be launched"); return -1; }
    return 0;
}

// Matrices with more weights than this go to the 32-row kernels instead (the library's own calls only): a stream that
// long is bound by the bytes in flight per compute unit, which LDS caps at 96 KB here.  Measured with 16 rows, both
// weight types: 14.7 M weights ([2048,7168]) 0.79-0.97 of the 32-row kernels' time, 29 M 1.09-1.12, 132 M 1.37-1.48.
// ZK_ROWS16_MAX_WEIGHTS overrides.
constexpr long kR16MaxWeights = 20L << 20;
static long r16_read_limit()
{
    const char *e = getenv("ZK_ROWS16_MAX_WEIGHTS");
    return e ? atol(e) : kR16MaxWeights;
}
static long g_r16_max_weights = r16_read_limit();
void gemm_rows16_reload_switches() { g_r16_max_weights = r16_read_limit(); }

// acc: scratch for split K (`max_slots` slots of 8 KB); null: the library's own, grown on demand
int gemm_rows16_launch(const GemmDesc &d, unsigned long long *acc, size_t max_slots)
{
    Rows16Params p;
    if (!r16_fill(d, p)) return 1;
    if (!acc && (long)d.N * d.K > g_r16_max_weights) return 1;
    std::lock_guard<std::mutex> lock(g_r16_mu);
    const long tiles = (long)d.G * p.row_tiles * p.col_groups;
    const long wg_tiles = (long)d.G * p.row_tiles * ((p.col_groups + kR16Waves - 1) / kR16Waves);
    if (tiles > (1L << 24)) return 1;
    const int slices = r16_slices(wg_tiles, d.K, r16_cus());
    if (slices > 1) {
        const size_t slots = (size_t)tiles * slices;
        if (acc) {
            // a caller's scratch: as many slices as its slots hold
            const long fit = (long)(max_slots / (size_t)tiles);
            const int use = slices < fit ? slices : (int)fit;
            if (use > 1) { p.acc = acc; p.nslices = use; }
        } else {
            const int rc = r16_scratch(slots);
            if (rc < 0) return -1;
            if (rc == 0) { p.acc = g_r16_acc; p.nslices = slices; }
        }
    }
    const int rc = r16_run(d.b32 ? gemm_rows16_kernel<true, false> : gemm_rows16_kernel<false, false>, p, wg_tiles * p.nslices);
    if (rc != 0 || p.nslices == 1) return rc;
    const long threads = tiles * (d.b32 ? R16Shape<true>::kColTiles : R16Shape<false>::kColTiles) * 4 * 64 * 4;      // four per output
    const dim3 grid((unsigned)((threads + 255) / 256));
    if (d.b32) gemm_rows16_finish_kernel<true><<<grid, dim3(256), 0, 0>>>(p);
    else gemm_rows16_finish_kernel<false><<<grid, dim3(256), 0, 0>>>(p);
    if (hipGetLastError() != hipSuccess) { set_error(kLaunchFailure, "gemm: the finishing kernel could not be launched"); return -1; }
    return 0;
}

int gemm_rows16_grouped(const GroupedDesc &d, const unsigned long long *guard)
{
    if (d.K < 0 || d.N < 1 || d.rows < 1 || d.groups < 1) return 1;
    std::lock_guard<std::mutex> lock(g_r16_mu);
    const int cols = d.b32 ? R16Shape<true>::kCols : R16Shape<false>::kCols;
    Rows16Params p = {};
    p.A = d.A; p.B = nullptr; p.C = d.C; p.R = d.R;
    p.lda = d.lda; p.sA = 0; p.ldb = d.K; p.sB = 0; p.ldc = d.ldc; p.sC = 0;
    p.G = 1; p.M = d.rows; p.N = d.N; p.K = d.K; p.shift = d.shift; p.b_shift = 0; p.init = d.init;
    p.row_tiles = 1;
    p.col_groups = (d.N + cols - 1) / cols;
    p.nslices = 1;
    p.grp_seg = d.seg; p.grp_tiles = d.tiles; p.grp_ntiles = d.ntiles; p.grp_b = d.B;
    p.guard = guard;
    // the grid covers the worst case of the tile table (the host never learns the segment sizes): rows / 32 + groups
    // tiles of 32 rows, two halves each
    const long blocks = ((long)d.rows / 32 + d.groups) * 2 * ((p.col_groups + kR16Waves - 1) / kR16Waves);
    return r16_run(d.b32 ? gemm_rows16_kernel<true, true> : gemm_rows16_kernel<false, true>, p, blocks);
}

}  // namespace zk

// ---- the entry point that allocates nothing -----------------------------------------------------------------
// Tight serving loops and harnesses that forbid it cannot call hipMalloc.  For them the
// scratch of the split-K launches is a file-scope device array: each GPU the library runs on holds its own copy, at its
// own address, until the process ends.  The array's name is a host-side stand-in, not a device address: its address on
// the current device is looked up once per device and that pointer is what the kernels get.
namespace zk {

constexpr size_t kNoAllocSlots = 1024;                                     // 8 MB: slots of 8 KB
static __device__ __align__(256) unsigned char scratch[kNoAllocSlots * kR16SlotBytes];

constexpr int kNoAllocMaxDevices = 64;
static unsigned long long *g_noalloc_ptr[kNoAllocMaxDevices] = {};

// the scratch array's address on the current device (null and an error recorded if it cannot be had)
static unsigned long long *noalloc_scratch(const char *name)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kNoAllocMaxDevices) {
        set_error(kLaunchFailure, "%s: cannot tell the current device", name);
        return nullptr;
    }
    if (!g_noalloc_ptr[dev]) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
            (void)hipGetLastError();
            set_error(kLaunchFailure, "%s: cannot find the scratch array on device %d", name, dev);
            return nullptr;
        }
        g_noalloc_ptr[dev] = reinterpret_cast<unsigned long long *>(ptr);
    }
    return g_noalloc_ptr[dev];
}

}  // namespace zk

extern "C" void int64_bmm_broadcast_noalloc(const int64_t *A, const void *B, int b32, int64_t *C, int64_t *R,
                                            int64_t b_rescale, int64_t c_rescale, int Bdim, int M, int K, int N)
{
    const char *name = "int64_bmm_broadcast_noalloc";
    using namespace zk;
    if (Bdim < 0 || M < 0 || K < 0 || N < 0) { set_error(kBadArgument, "%s: negative dimension", name); return; }
    if (c_rescale < 0 || c_rescale > 63) { set_error(kBadArgument, "%s: shift %lld outside [0,63]", name, (long long)c_rescale); return; }
    if (b_rescale <= 0 || (b_rescale & (b_rescale - 1)) != 0) {
        set_error(kBadArgument, "%s: the divisor of B must be a positive power of two", name);
        return;
    }
    if (M > kNoAllocMaxRows) { set_error(kUnsupportedSize, "%s: %d rows, at most %d", name, M, kNoAllocMaxRows); return; }
    if (Bdim == 0 || M == 0 || N == 0) return;
    // (each factor on its own first: the product of three ints can leave 64 bits)
    if (Bdim > kNoAllocMaxOutputs || N > kNoAllocMaxOutputs || (long)Bdim * M > kNoAllocMaxOutputs || (long)Bdim * M * N > kNoAllocMaxOutputs) {
        set_error(kUnsupportedSize, "%s: %d x %d x %d outputs, at most %ld", name, Bdim, M, N, kNoAllocMaxOutputs);
        return;
    }
    if (!A || !B || !C) { set_error(kBadArgument, "%s: null pointer", name); return; }
    unsigned long long *ptr = noalloc_scratch(name);
    if (!ptr) return;
    GemmDesc d;
    d.A = A; d.lda = K; d.sA = (long)M * K;
    d.B = B; d.b32 = b32 ? 1 : 0; d.ldbn = K; d.ldbk = 1; d.sB = 0;
    d.C = C; d.R = R; d.ldc = N; d.sC = (long)M * N;
    d.G = Bdim; d.M = M; d.N = N; d.K = K;
    d.shift = (int)c_rescale; d.init = 0; d.a_rs = 1; d.b_rs = b_rescale;
    // (a K split that would need more slots than the array has is cut down to what fits; one slice needs none)
    if (gemm_rows16_launch(d, ptr, kNoAllocSlots) == 1) set_error(kUnsupportedSize, "%s: shape outside what the 16-row kernels take", name);
}

