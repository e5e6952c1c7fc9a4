// Grouped product on 32-row tiles with int32 weights, the weights streamed through LDS rings
// (see gemm_mfma.hip for the digit scheme and gemm_mfma_grouped for the launch this kernel is one form of).
//
// The routed experts of a MoE layer are a stream over their weights: an expert has a handful of rows, so the matrix
// work is small next to the one pass over 45 GB of int32.  The general 32-row kernel stages a step of B in registers,
// splits it and hands the digits to the other wavefronts through LDS; its next loads can leave only when the staging
// registers are free again, so every step pays a load's latency plus the split.  Here a wavefront owns 32 columns
// outright: their raw elements travel from global memory straight into a ring in LDS (global_load_lds_dwordx4: no
// register is held while a load is under way, three steps are under way at any time), the lanes read them back in
// the order the matrix instruction wants, split them in registers and multiply.  Nothing of B is shared, so B needs
// no barrier; the 32 rows of A are shared: every wavefront streams an eighth of them the same way, splits its
// eighth and leaves the digits in LDS for all (one barrier per step).
//
// Reading back in fragment order without bank conflicts.  Lane (n, h) = (lane % 32, lane / 32) of the B operand of
// v_mfma_i32_32x32x32_i8 holds k = 16h .. 16h+15 of column n: four 16-byte chunks (4h + j, j = 0..3) of the 128 bytes a
// row has per step.  A load instruction q (0..3) covers rows 8q .. 8q+7, eight lanes per row (128 contiguous bytes),
// and lane l lands at byte 16 l of the instruction's 1 KB block.  Lane 8r + c of instruction q loads chunk
// (c & 4) | ((c ^ q) & 3) of row 8q + r, so chunk 4h + j of row n sits at slot 8 (n % 8) + 4h + (j ^ (n / 8)) of block
// n / 8: for a fixed j the 64 lanes of a read hit 64 different slots.
//
// Tiles of at most 16 rows (nearly every tile of a routed expert) multiply on v_mfma_i32_16x16x64_i8 over pairs of steps:
// half the matrix work for the same bytes, which on this power-managed device is what lets the stream run faster.  For
// the same reason rows past the end of a segment are multiplied as zeros, not as copies of its last row.
#pragma once
#include "lds_dma.h"

namespace zk {

constexpr int kS32Stages = 3;            // steps of raw elements under way per wavefront
constexpr int kS32Loads = 5;             // loads per wavefront and step: one piece of A, four of B

constexpr size_t stream32_lds_bytes(int na) { return (size_t)kS32Stages * (8 * 4096 + 8192) + 2 * (size_t)na * 1024; }

template <int NA, int NB>
__global__ __launch_bounds__(512) void gemm_stream32_grouped_kernel(MfmaParams p)
{
    constexpr int D = NA + NB - 1;
    constexpr int STG = kS32Stages;
    extern __shared__ __attribute__((aligned(16))) unsigned char s32_smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    unsigned char *ring_b = s32_smem + wave * (STG * 4096);                  // [stage][instruction][lane] 16 bytes
    unsigned char *ring_a = s32_smem + 8 * STG * 4096;                       // [stage][wavefront][lane] 16 bytes
    unsigned char *adig = ring_a + STG * 8192;                               // [2][digit][1 KB], fragment order
    const unsigned ring_b_lds = (unsigned)(uintptr_t)ring_b, ring_a_lds = (unsigned)(uintptr_t)ring_a + wave * 1024;

    // (the tile columns of one 32-row tile on one XCD, as in gemm_mfma_block's grouped form: its rows of A come from memory once)
    const int xcd = (int)blockIdx.x & 7, w = (int)blockIdx.x >> 3, wq = w / p.tiles_n;
    const int mt = wq * 8 + xcd;
    unsigned long long *slot = p.wg_range + 4 * (long)blockIdx.x;
    if (mt >= *p.grp_ntiles) {                   // the grid covers the worst case: nothing to do, an empty range
        if (tid == 0) { slot[0] = ~0ull; slot[1] = 0ull; slot[2] = ~0ull; slot[3] = 0ull; }
        return;
    }
    const int tn = w - wq * p.tiles_n;
    const int e = p.grp_tiles[2 * mt];
    const int m0 = p.grp_tiles[2 * mt + 1], m_lim = p.grp_seg[e + 1];
    const int32_t *b_base = reinterpret_cast<const int32_t *>(p.grp_b[e]);
    if ((uintptr_t)b_base & 15) {
        // a matrix that does not start on a 16-byte boundary: the loads into LDS cannot take it.  The workgroup reports
        // the full range for B instead of computing (and nothing for A, which it has not looked at): no digit count
        // covers that, so the guarded launch behind this one (or the caller's next route) computes these outputs.
        if (tid == 0) { slot[0] = ~0ull; slot[1] = 0ull; slot[2] = 0ull; slot[3] = ~0ull; }
        return;
    }
    const int n0 = tn * 256 + wave * 32;
    const int ksteps = p.K / 32;

    // ---- what this lane loads ----
    const int32_t *bq[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int r = lane >> 3, c = lane & 7;
        int n = n0 + 8 * q + r;
        n = n < p.N ? n : p.N - 1;               // columns past N: any valid data, never stored
        bq[q] = b_base + (long)n * p.ldbn + 4 * ((c & 4) | ((c ^ q) & 3));
    }
    const int a_r = 4 * wave + (lane >> 4), a_c = lane & 15;                 // row of the tile, pair of k
    int am = m0 + a_r;
    // Rows past the end of the segment are loaded from its last row (a valid address) but multiplied as ZEROS: an expert
    // has some 8 of the tile's 32 rows, and what the matrix pipe draws depends on the bits it is fed.  The device is
    // power managed, so three quarters of the products running on copies of real rows slowed the whole stream down
    // (int32 experts, (4,4) digits: 4.85 TB/s with copies, 5.7 with zeros).
    const bool a_pad = am >= m_lim;
    am = am < m_lim ? am : m_lim - 1;
    const int64_t *a_src = p.A + (long)am * p.lda + 2 * a_c;
    // where this lane's two digits of A go in a digit block, and what it reads back of B
    const int a_dst = (a_r + 32 * (a_c >> 3)) * 16 + 2 * (a_c & 7);
    const int n_l = lane & 31, h_l = lane >> 5;
    int b_rd[4];
#pragma unroll
    for (int j = 0; j < 4; j++) b_rd[j] = (n_l >> 3) * 1024 + (8 * (n_l & 7) + 4 * h_l + ((j ^ (n_l >> 3)) & 3)) * 16;

    // step t on its way: this wavefront's eighth of A for step t + 1 and its own columns for step t
    auto issue = [&](int t) {
        const unsigned st = (unsigned)(t % STG);
        const int ta = t + 1 < ksteps ? t + 1 : t;
        lds_dma16(a_src + 32 * (long)ta, ring_a_lds + st * 8192);
#pragma unroll
        for (int q = 0; q < 4; q++) lds_dma16(bq[q] + 32 * (long)t, ring_b_lds + st * 4096 + q * 1024);
    };

    // ---- range tracking (see gemm_mfma_block): A is shared out over the first tile columns, B is all this workgroup's ----
    const int vmod_a = p.tiles_n < 8 ? p.tiles_n : 8;
    const bool verify_a = tn < vmod_a;
    DigitsSeen oa;
    int rb_lo = INT32_MAX, rb_hi = INT32_MIN;
    int turn_a = 0;                              // step % vmod_a of the step whose rows are split next

    // two elements of A (k = 2c, 2c + 1 of this lane's row) -> their NA digits into digit blocks of `stage`
    // (called once per step, in order)
    auto stash_a = [&](const v4i &raw, int stage) {
        const int64_t x0 = (int64_t)(((uint64_t)(uint32_t)raw[1] << 32) | (uint32_t)raw[0]);
        const int64_t x1 = (int64_t)(((uint64_t)(uint32_t)raw[3] << 32) | (uint32_t)raw[2]);
        if (verify_a && turn_a == tn) { oa.add(x0); oa.add(x1); oa.seen = true; }
        turn_a = turn_a + 1 == vmod_a ? 0 : turn_a + 1;
        const uint64_t u0 = ((uint64_t)x0 + Limb<NA>::kBias) ^ Limb<NA>::kBias, u1 = ((uint64_t)x1 + Limb<NA>::kBias) ^ Limb<NA>::kBias;
        unsigned char *dst = adig + stage * (NA * 1024) + a_dst;
#pragma unroll
        for (int i = 0; i < NA; i++) {
            const uint32_t d0 = (uint32_t)(u0 >> (8 * i)) & 0xFFu, d1 = (uint32_t)(u1 >> (8 * i)) & 0xFFu;
            *reinterpret_cast<uint16_t *>(dst + i * 1024) = a_pad ? (uint16_t)0 : (uint16_t)(d0 | (d1 << 8));
        }
    };

    // prologue: the digits of A for step 0 straight from memory, the first steps on their way
    {
        const v4i a0 = *(const ZK_GLOBAL_MEM v4i *)(a_src);
        stash_a(a0, 0);
    }
#pragma unroll
    for (int d = 0; d < STG; d++)
        if (d < ksteps) issue(d);
    __syncthreads();

    // what every step begins with: its stage has landed (the loads of later steps may still be under way)
    auto landed = [&](int s) {
        const int behind = ksteps - 1 - s;
        if (behind >= 2) wait_vmcnt<2 * kS32Loads>();
        else if (behind == 1) wait_vmcnt<kS32Loads>();
        else wait_vmcnt<0>();
        asm volatile("" ::: "memory");                     // (the reads that follow stay behind the wait)
    };
    auto track_b = [&](const v4i &v) {
#pragma unroll
        for (int z = 0; z < 4; z++) {
            rb_lo = v[z] < rb_lo ? v[z] : rb_lo;
            rb_hi = v[z] > rb_hi ? v[z] : rb_hi;
        }
    };
    const uint64_t rmask = p.shift ? ((1ull << p.shift) - 1) : 0;
    const int sh = p.shift;
    // diagonals of one output -> 128-bit sum -> shift -> C and R (diagonals are added in 64-bit groups of four, the groups
    // meet in 128 bits)
    auto finish = [&](const int (&dg)[D], int m, int n) {
        u128 sum = (u128)(i128)p.init;
#pragma unroll
        for (int gq = 0; gq < (D + 3) / 4; gq++) {
            uint64_t sg = (uint64_t)(int64_t)dg[4 * gq];
#pragma unroll
            for (int j = 1; j < 4; j++)
                if (4 * gq + j < D) sg += (uint64_t)(int64_t)dg[4 * gq + j] << (8 * j);
            sum += (u128)(i128)(int64_t)sg << (32 * gq);
        }
        if (!(m < m_lim && n < p.N)) return;
        const uint64_t lo = (uint64_t)sum, hi = (uint64_t)(sum >> 64);
        const long o = (long)m * p.ldc + n;
        p.C[o] = (int64_t)((lo >> sh) | ((hi << 1) << (63 - sh)));
        if (p.R) p.R[o] = (int64_t)(lo & rmask);
    };

    if (m_lim - m0 <= 16) {
        // ---- at most 16 rows (nearly every tile of a routed expert): v_mfma_i32_16x16x64_i8, half the matrix work ----
        // Lane (i, q) = (lane % 16, lane / 16) of either operand holds k = 16q .. 16q+15 of a pair of steps for row i of
        // A, or for column 16 ct + i of B (ct = 0, 1: the wavefront's two column tiles).  That is half q % 2 of step
        // 2u + q / 2: a lane reads at the steps of its own parity only and keeps what it read; the products follow at
        // the odd steps (and at a last even one, where the lanes of the missing step hold zeros for A).
        const int li = lane & 15, lq = lane >> 4;
        const bool odd_lane = (lq >> 1) != 0;
        int b_rd16[2][4];
#pragma unroll
        for (int ct = 0; ct < 2; ct++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int nn = 16 * ct + li;
                b_rd16[ct][j] = (nn >> 3) * 1024 + (8 * (nn & 7) + 4 * (lq & 1) + ((j ^ (nn >> 3)) & 3)) * 16;
            }
        const int a_rd16 = (li + 32 * (lq & 1)) * 16;
        v4i acc[D][2];
#pragma unroll
        for (int d = 0; d < D; d++)
#pragma unroll
            for (int ct = 0; ct < 2; ct++) acc[d][ct] = v4i{ 0, 0, 0, 0 };
        v4i raw[2][4], fa[NA];
#pragma unroll
        for (int i = 0; i < NA; i++) fa[i] = v4i{ 0, 0, 0, 0 };
#pragma unroll
        for (int ct = 0; ct < 2; ct++)
#pragma unroll
            for (int j = 0; j < 4; j++) raw[ct][j] = v4i{ 0, 0, 0, 0 };

        for (int s = 0; s < ksteps; s++) {
            landed(s);
            const unsigned st = (unsigned)(s % STG);
            const bool mine = odd_lane == ((s & 1) != 0);
            if (mine) {
#pragma unroll
                for (int ct = 0; ct < 2; ct++)
#pragma unroll
                    for (int j = 0; j < 4; j++) raw[ct][j] = *reinterpret_cast<const v4i *>(ring_b + st * 4096 + b_rd16[ct][j]);
#pragma unroll
                for (int i = 0; i < NA; i++) fa[i] = *reinterpret_cast<const v4i *>(adig + (s & 1) * (NA * 1024) + i * 1024 + a_rd16);
            }
            const v4i araw = *reinterpret_cast<const v4i *>(ring_a + st * 8192 + wave * 1024 + lane * 16);
            if (s + STG < ksteps) {
                __builtin_amdgcn_s_waitcnt(0xC07F);        // lgkmcnt(0): the reads above have returned before their stage is overwritten
                issue(s + STG);
            }
            if (mine) {
#pragma unroll
                for (int ct = 0; ct < 2; ct++)
#pragma unroll
                    for (int j = 0; j < 4; j++) track_b(raw[ct][j]);
            }
            if (s + 1 < ksteps) stash_a(araw, (s + 1) & 1);
            const bool last_even = s + 1 == ksteps && !(s & 1);
            if ((s & 1) || last_even) {
                if (last_even && odd_lane) {               // no step 2u + 1: these lanes multiply zeros
#pragma unroll
                    for (int i = 0; i < NA; i++) fa[i] = v4i{ 0, 0, 0, 0 };
                }
#pragma unroll
                for (int ct = 0; ct < 2; ct++) {
                    int x[16];
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int z = 0; z < 4; z++) x[4 * j + z] = raw[ct][j][z];
                    v4i fb[NB];
                    split16_w32<NB>(x, fb);
#pragma unroll
                    for (int i = 0; i < NA; i++)
#pragma unroll
                        for (int j = 0; j < NB; j++)
                            acc[i + j][ct] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[i], fb[j], acc[i + j][ct], 0, 0, 0);
                }
            }
            __syncthreads();
        }
        // accumulator register r of lane l holds row 4 (l / 16) + r, column l % 16 of its column tile
#pragma unroll
        for (int ct = 0; ct < 2; ct++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                int dg[D];
#pragma unroll
                for (int d = 0; d < D; d++) dg[d] = acc[d][ct][r];
                finish(dg, m0 + 4 * lq + r, n0 + 16 * ct + li);
            }
    } else {
        v16i acc[D];
#pragma unroll
        for (int d = 0; d < D; d++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[d][r] = 0;

        for (int s = 0; s < ksteps; s++) {
            landed(s);
            const unsigned st = (unsigned)(s % STG);
            v4i raw[4], araw, fa[NA];
#pragma unroll
            for (int j = 0; j < 4; j++) raw[j] = *reinterpret_cast<const v4i *>(ring_b + st * 4096 + b_rd[j]);
            araw = *reinterpret_cast<const v4i *>(ring_a + st * 8192 + wave * 1024 + lane * 16);
#pragma unroll
            for (int i = 0; i < NA; i++) fa[i] = *reinterpret_cast<const v4i *>(adig + (s & 1) * (NA * 1024) + i * 1024 + lane * 16);
            if (s + STG < ksteps) {
                __builtin_amdgcn_s_waitcnt(0xC07F);        // lgkmcnt(0): the reads above have returned before their stage is overwritten
                issue(s + STG);
            }
            // the weights of this step: range, digits
            int x[16];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                track_b(raw[j]);
#pragma unroll
                for (int z = 0; z < 4; z++) x[4 * j + z] = raw[j][z];
            }
            v4i fb[NB];
            split16_w32<NB>(x, fb);
            // this wavefront's eighth of A for the next step
            if (s + 1 < ksteps) stash_a(araw, (s + 1) & 1);
#pragma unroll
            for (int i = 0; i < NA; i++)
#pragma unroll
                for (int j = 0; j < NB; j++)
                    acc[i + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i + j], 0, 0, 0);
            __syncthreads();
        }
        // accumulator register r of lane l holds row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32
#pragma unroll
        for (int r = 0; r < 16; r++) {
            int dg[D];
#pragma unroll
            for (int d = 0; d < D; d++) dg[d] = acc[d][r];
            finish(dg, m0 + 4 * (lane >> 5) + 8 * (r >> 2) + (r & 3), n0 + (lane & 31));
        }
    }

    // every workgroup leaves its ranges in its own slot; the waves' ranges meet in LDS (the rings are free by now)
    MinMax ra = oa.range(), rb = { INT64_MAX, INT64_MIN };
    if (rb_lo <= rb_hi) rb = MinMax{ (int64_t)rb_lo, (int64_t)rb_hi };
    ra = mm_wave(ra);
    rb = mm_wave(rb);
    MinMax *red = reinterpret_cast<MinMax *>(s32_smem);
    if (lane == 0) { red[2 * wave] = ra; red[2 * wave + 1] = rb; }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 8; w++) { mm_merge(ra, red[2 * w]); mm_merge(rb, red[2 * w + 1]); }
        slot[0] = (unsigned long long)ra.lo ^ kSignFlip;
        slot[1] = (unsigned long long)ra.hi ^ kSignFlip;
        slot[2] = (unsigned long long)rb.lo ^ kSignFlip;
        slot[3] = (unsigned long long)rb.hi ^ kSignFlip;
    }
}

// the kernel for digit counts (na, nb), or null; *lds receives its dynamic LDS size
MfmaKernel stream32_grouped_kernel(int na, int nb, size_t *lds);

}  // namespace zk
