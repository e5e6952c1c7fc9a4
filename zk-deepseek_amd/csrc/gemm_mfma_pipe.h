// 128 x 128 tiles with BOTH operands from digit planes (A pre-split by the pass in front, B prepared once): nothing is
// split, tracked or staged in registers, so the step is loads, fragment reads and MFMAs only, and it is written as a
// software pipeline instead of the fenced phases of gemm_mfma_block:
//   * the planes of a step are 4 (NA + NB) blocks of 1 KB, already in fragment order; every wavefront sends its share of
//     them from global memory straight into a ring of LDS stages (global_load_lds_dwordx4), kPipeStages - 1 steps before
//     they are multiplied, one load at a time between MFMAs;
//   * the fragments of step s+1 are read into registers while the MFMAs of step s run: B's into a second set of
//     registers at the start of the step, A's digit by digit into the registers whose last use has just been issued
//     (the MFMAs go through A's digits in order), so that the matrix pipe has its operands the moment the step's one
//     barrier opens.
// Eight wavefronts as 2 x 4, 64 x 32 outputs each, as in the general kernel; tiles, split tail tiles, partial sums, range
// slots and outputs are the general kernel's (gemm_mfma_block with APL and BPL), which this one replaces for three digits
// a side.
#pragma once
#include "lds_dma.h"

namespace zk {

constexpr int kPipeStages = 5;

constexpr size_t pipe_lds_bytes(int na, int nb) { return (size_t)kPipeStages * 4 * (size_t)(na + nb) * 1024; }

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>());
        static_for<I + 1, N>(f);
    }
}

template <int NA, int NB>
__global__ __launch_bounds__(512) void gemm_mfma_pipe_kernel(MfmaParams p)
{
    constexpr int D = NA + NB - 1, STG = kPipeStages, AHEAD = STG - 1, T = 512;
    constexpr int BLOCKS = 4 * (NA + NB), STAGE = BLOCKS * 1024;
    constexpr int LOADS = BLOCKS / 8;                       // per wavefront and step
    static_assert(D <= 5, "160 accumulator registers: two wavefronts share a SIMD");
    static_assert(BLOCKS % 8 == 0, "every wavefront loads the same number of blocks");
    static_assert(LOADS * (AHEAD - 1) < 64, "vmcnt is a 6-bit counter");
    extern __shared__ __attribute__((aligned(16))) unsigned char pipe_smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);            // (the same in every lane)
    const int wm = wave >> 2, wn = wave & 3;
    const unsigned ring_lds = (unsigned)(uintptr_t)pipe_smem;

    // workgroup -> tile or slice of a split tile, as in gemm_mfma_block
    const int per_batch = p.tiles_m * p.tiles_n;
    int lin = (int)blockIdx.x, sidx = 0, nsplit = 1;
    if (lin < p.main_tiles) {
        if ((p.main_tiles & 7) == 0) lin = (lin & 7) * (p.main_tiles >> 3) + (lin >> 3);
    } else {
        const int t = lin - p.main_tiles;
        if (p.tail_xcd) {
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
    const int tail_tile = lin - p.main_tiles;
    const int g = lin / per_batch, rem = lin - g * per_batch;
    int tm, tn;
    if (p.n_fastest) { tm = rem / p.tiles_n; tn = rem - tm * p.tiles_n; }
    else { tn = rem / p.tiles_m; tm = rem - tn * p.tiles_m; }
    const int m0 = tm * 128, n0 = tn * 128, m_lim = p.M;
    const int ksteps = (p.K + 31) / 32;                     // (the planes are padded with zeros to whole steps)
    const int ks_begin = (int)((long)sidx * ksteps / nsplit), ks_end = (int)((long)(sidx + 1) * ksteps / nsplit);
    const int nsteps = ks_end - ks_begin;

    // ---- this wavefront's blocks of a step: numbers wave * LOADS + l of [A: 32-row group 0..3][digit], [B: 32-column group 0..3][digit] ----
    const unsigned char *src[LOADS];
    long stride[LOADS];
#pragma unroll
    for (int l = 0; l < LOADS; l++) {
        const int b = wave * LOADS + l;
        if (b < 4 * NA) {
            const int grp = b / NA, dig = b - grp * NA;
            src[l] = p.a_planes + ((((long)g * p.a_msub + (m0 >> 5) + grp) * p.a_ksteps + ks_begin) * NA + dig) * 1024 + lane * 16;
            stride[l] = NA * 1024;
        } else {
            const int bb = b - 4 * NA, grp = bb / NB, dig = bb - grp * NB;
            int sub = (n0 >> 5) + grp;
            sub = sub < p.b_nsub ? sub : p.b_nsub - 1;      // column groups past N: any valid data, never stored
            src[l] = reinterpret_cast<const unsigned char *>(p.B) + (((long)sub * p.b_ksteps + ks_begin) * NB + dig) * 1024 + lane * 16;
            stride[l] = NB * 1024;
        }
    }
    auto issue_one = [&](int t, auto l_tag) {               // load l of local step t
        constexpr int L = decltype(l_tag)::value;
        const int tc = t < nsteps ? t : nsteps - 1;         // (past the end: the last step again, into a stage nobody reads any more)
        lds_dma16(src[L] + (long)tc * stride[L], ring_lds + (unsigned)(t % STG) * STAGE + (wave * LOADS + L) * 1024);
    };
    auto issue = [&](int t) { static_for<0, LOADS>([&](auto l) { issue_one(t, l); }); };

    v16i acc[2][D];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int d = 0; d < D; d++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][d][r] = 0;

    auto read_a = [&](unsigned st, int a, int i) {
        return *reinterpret_cast<const v4i *>(pipe_smem + st * STAGE + ((wm * 2 + a) * NA + i) * 1024 + lane * 16);
    };
    auto read_b = [&](unsigned st, int j) {
        return *reinterpret_cast<const v4i *>(pipe_smem + st * STAGE + (4 * NA + wn * NB + j) * 1024 + lane * 16);
    };

    // prologue: AHEAD steps under way, the first one's fragments in registers
#pragma unroll
    for (int t = 0; t < AHEAD; t++) issue(t);
    wait_vmcnt<LOADS * (AHEAD - 1)>();                     // step 0 has landed (my share)
    asm volatile("" ::: "memory");
    __syncthreads();
    v4i fa[2][NA], fb[NB];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int i = 0; i < NA; i++) fa[a][i] = read_a(0, a, i);
#pragma unroll
    for (int j = 0; j < NB; j++) fb[j] = read_b(0, j);

    // Step s: the MFMAs of step s on the fragments in registers; beside them the fragment reads of step s+1 (landed and
    // fenced by the barrier at the top) and the loads of step s+AHEAD into the stage step s-1 was read from (those reads
    // were waited for by the MFMAs of step s-1).
    static_assert((NA - 1) * NB >= LOADS, "the loads ride behind the MFMAs of A's digits from the second on");
    for (int s = 0; s < nsteps; s++) {
        wait_vmcnt<LOADS * (AHEAD - 2)>();                  // step s+1 has landed (my share): steps s+2 .. s+AHEAD-1 may be under way
        asm volatile("" ::: "memory");
        __syncthreads();
        const unsigned sn = (unsigned)((s + 1) % STG);
        v4i fbn[NB];
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, NA>([&](auto i_tag) {
            constexpr int I = decltype(i_tag)::value;
            static_for<0, NB>([&](auto j_tag) {
                constexpr int J = decltype(j_tag)::value;
#pragma unroll
                for (int a = 0; a < 2; a++) acc[a][I + J] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[a][I], fb[J], acc[a][I + J], 0, 0, 0);
                // behind the first digit's MFMAs: the next step's fragments of B; behind the others': the loads, one at a time
                if constexpr (I == 0) fbn[J] = read_b(sn, J);
                constexpr int L = (I - 1) * NB + J;
                if constexpr (I >= 1 && L < LOADS) {
                    __builtin_amdgcn_sched_barrier(0);
                    issue_one(s + AHEAD, std::integral_constant<int, (I >= 1 && L < LOADS) ? L : 0>());
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            // digit I of A has been issued for the last time this step: its registers take the next step's
            fa[0][I] = read_a(sn, 0, I);
            fa[1][I] = read_a(sn, 1, I);
            __builtin_amdgcn_sched_barrier(0);
        });
#pragma unroll
        for (int j = 0; j < NB; j++) fb[j] = fbn[j];
    }
    wait_vmcnt<0>();                                       // (the loads past the end)
    asm volatile("" ::: "memory");

    // both operands' ranges were fixed when their planes were written: an empty range from here
    if (tid == 0) {
        unsigned long long *slot = p.wg_range + 4 * (long)blockIdx.x;
        slot[0] = ~0ull; slot[1] = 0ull; slot[2] = ~0ull; slot[3] = 0ull;
    }

    // epilogue: diagonals -> 128-bit sum -> shift, as in gemm_mfma_block (accumulator register r of lane l holds
    // row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its 32 x 32 tile)
    auto combine = [&](int a, int r, u128 sum) {
#pragma unroll
        for (int gq = 0; gq < (D + 3) / 4; gq++) {
            uint64_t sg = (uint64_t)(int64_t)acc[a][4 * gq][r];
#pragma unroll
            for (int j = 1; j < 4; j++)
                if (4 * gq + j < D) sg += (uint64_t)(int64_t)acc[a][4 * gq + j][r] << (8 * j);
            sum += (u128)(i128)(int64_t)sg << (32 * gq);
        }
        return sum;
    };
    if (nsplit > 1) {
        // raw partial sums in the layout gemm_split_finish_kernel<2, 4, 2, 1> adds up
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                if (m0 + (wm * 2 + a) * 32 + 8 * (r >> 2) + (r & 3) >= m_lim) continue;
                const u128 sum = combine(a, r, 0);
                const long q = (((long)tail_tile * p.split + sidx) * (T / 64) + wave) * 32 + a * 16 + r;
                if (p.part64) p.partials[q * 64 + lane] = (uint64_t)sum;
                else { p.partials[q * 128 + lane] = (uint64_t)sum; p.partials[q * 128 + 64 + lane] = (uint64_t)(sum >> 64); }
            }
        return;
    }
    const uint64_t rmask = p.shift ? ((1ull << p.shift) - 1) : 0;
    const u128 sum0 = (u128)(i128)p.init;
    const int sh = p.shift;
    auto store_tile = [&](auto edge_tag, auto rem_tag) {
        constexpr bool EDGE = decltype(edge_tag)::value, REM = decltype(rem_tag)::value;
        const int n = n0 + wn * 32 + (lane & 31);
#pragma unroll
        for (int a = 0; a < 2; a++) {
            const int mrow = m0 + (wm * 2 + a) * 32 + 4 * (lane >> 5);
            const long o0 = (long)g * p.sC + (long)mrow * p.ldc + n;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int dr = 8 * (r >> 2) + (r & 3);
                const u128 sum = combine(a, r, sum0);
                const uint64_t lo = (uint64_t)sum, hi = (uint64_t)(sum >> 64);
                if (EDGE && !(mrow + dr < m_lim && n < p.N)) continue;
                const long o = o0 + (long)dr * p.ldc;
                p.C[o] = (int64_t)((lo >> sh) | ((hi << 1) << (63 - sh)));
                if (REM) p.R[o] = (int64_t)(lo & rmask);
            }
        }
    };
    const bool edge = m0 + 128 > m_lim || n0 + 128 > p.N;
    if (p.R) { if (edge) store_tile(std::true_type(), std::true_type()); else store_tile(std::false_type(), std::true_type()); }
    else { if (edge) store_tile(std::true_type(), std::false_type()); else store_tile(std::false_type(), std::false_type()); }
}

// the kernel for digit counts (na, nb), or null, and its dynamic LDS
MfmaKernel pipe_kernel(int na, int nb);
size_t pipe_lds_size(int na, int nb);

}  // namespace zk
