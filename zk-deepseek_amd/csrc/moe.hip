// Dispatch of a MoE layer on the device: tokens sorted by expert, the grouped expert GEMM, the weighted combine.
//
// The reference loops over the experts in Python (MoE.forward, inference/model.py:1325-1383): torch.where per
// expert, three GEMM calls on a handful of tokens each, index_add.  Here the routing result stays on the device:
// moe_dispatch sorts the (token, slot) entries by expert (stable, so every expert sees its tokens in ascending
// order like torch.where gives them), int64_grouped_bmm_launcher runs one GEMM launch over all experts, and
// moe_combine adds floor(y_expert * weight / 2^shift) over the slots of every token.
#include "gemm.h"
#include "../../include/int64gemm.h"

#include <vector>

namespace zk {

// entries = T * K routed (token, slot) pairs, entry i = token i / K, slot i % K, expert indices[i]

__global__ __launch_bounds__(256) void moe_count_kernel(const int64_t *__restrict__ indices, long entries, int *__restrict__ counts)
{
    __shared__ int red[4];
    const int e = blockIdx.x;
    int c = 0;
    for (long i = threadIdx.x; i < entries; i += 256) c += indices[i] == e ? 1 : 0;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off, kWave);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) counts[e] = red[0] + red[1] + red[2] + red[3];
}

// exclusive scan of the counts and the table of 32-row tiles: one workgroup, 256 experts per round (a single thread
// walking 256 counts took 19 us, longer than every other step of a one-token dispatch)
// Entries whose expert index lies outside [0, E) are counted by no workgroup: the rows behind the last segment then
// belong to nobody.  Their tokens are set to 0 here (so that a gather reads valid memory) and `bad_host`, a flag in
// pinned host memory, reports the call.
__global__ __launch_bounds__(256) void moe_scan_kernel(const int *__restrict__ counts, int E, int *__restrict__ seg, int *__restrict__ tiles,
                                                       int *__restrict__ ntiles, long entries, int *__restrict__ sorted_token,
                                                       int *bad_host)
{
    __shared__ int wave_sum[2][4];
    __shared__ int carry[2];                       // rows and tiles of the rounds before this one
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) carry[0] = carry[1] = 0;
    __syncthreads();
    for (int e0 = 0; e0 < E; e0 += 256) {
        const int e = e0 + (int)threadIdx.x;
        const int c = e < E ? counts[e] : 0, t = (c + 31) >> 5;
        int pc = c, pt = t;                        // inclusive prefix sums over the wave
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int vc = __shfl_up(pc, off, 64), vt = __shfl_up(pt, off, 64);
            if (lane >= off) { pc += vc; pt += vt; }
        }
        if (lane == 63) { wave_sum[0][wave] = pc; wave_sum[1][wave] = pt; }
        __syncthreads();
        int bc = carry[0], bt = carry[1];
        for (int w = 0; w < wave; w++) { bc += wave_sum[0][w]; bt += wave_sum[1][w]; }
        if (e < E) {
            const int row = bc + pc - c, tile = bt + pt - t;
            seg[e] = row;
            for (int i = 0; i < t; i++) { tiles[2 * (tile + i)] = e; tiles[2 * (tile + i) + 1] = row + 32 * i; }
        }
        __syncthreads();
        if (threadIdx.x == 255) { carry[0] = bc + pc; carry[1] = bt + pt; }
        __syncthreads();
    }
    const int placed = carry[0];
    if (threadIdx.x == 0) { seg[E] = placed; ntiles[0] = carry[1]; }
    for (long r = placed + (long)threadIdx.x; r < entries; r += 256) sorted_token[r] = 0;
    if (threadIdx.x == 0 && placed != entries && bad_host) *bad_host = 1;
}

// workgroup e walks the entries in order and gives its own consecutive rows: a stable partition
__global__ __launch_bounds__(256) void moe_place_kernel(const int64_t *__restrict__ indices, long entries, int K,
                                                        const int *__restrict__ seg, int *__restrict__ sorted_token,
                                                        int *__restrict__ sorted_pos)
{
    __shared__ int wave_count[4];
    __shared__ int base_s;
    const int e = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) base_s = seg[e];
    __syncthreads();
    for (long start = 0; start < entries; start += 256) {
        const long i = start + threadIdx.x;
        const int64_t idx = i < entries ? indices[i] : -1;
        const bool mine = i < entries && idx == e;
        // an index outside [0, E) belongs to no workgroup: its entry points at row 0 rather than at whatever the buffer held
        if (e == 0 && i < entries && (idx < 0 || idx >= (int64_t)gridDim.x)) sorted_pos[i] = 0;
        const unsigned long long ballot = __ballot(mine);
        const int before = __popcll(ballot & ((1ull << lane) - 1));
        if (lane == 0) wave_count[wave] = __popcll(ballot);
        __syncthreads();
        int offset = base_s;
        for (int w = 0; w < wave; w++) offset += wave_count[w];
        if (mine) {
            const int r = offset + before;
            sorted_token[r] = (int)(i / K);
            sorted_pos[i] = r;
        }
        __syncthreads();
        if (threadIdx.x == 0) base_s += wave_count[0] + wave_count[1] + wave_count[2] + wave_count[3];
        __syncthreads();
    }
}

struct __attribute__((aligned(16))) i64x2m { int64_t x, y; };

// out[r][:] = x[token[r]][:]
__global__ __launch_bounds__(256) void moe_gather_kernel(const int64_t *__restrict__ x, const int *__restrict__ token,
                                                         int64_t *__restrict__ out, int N, int vec)
{
    const long r = blockIdx.y;
    const int64_t *src = x + (long)token[r] * N;
    int64_t *dst = out + r * N;
    if (vec) {
        for (int i = (blockIdx.x * 256 + threadIdx.x) * 2; i < N; i += gridDim.x * 512)
            *reinterpret_cast<i64x2m *>(dst + i) = *reinterpret_cast<const i64x2m *>(src + i);
    } else {
        for (int i = blockIdx.x * 256 + threadIdx.x; i < N; i += gridDim.x * 256) dst[i] = src[i];
    }
}

// y[t][n] = sum_k (ye[pos[t][k]][n] * w[t][k]) >> shift   (wrapping products and sums, floor shift: model.py:1379)
__global__ __launch_bounds__(256) void moe_combine_kernel(const int64_t *__restrict__ ye, const int64_t *__restrict__ w,
                                                          const int *__restrict__ pos, int64_t *__restrict__ y, int K, int N,
                                                          int shift)
{
    const long t = blockIdx.y;
    for (int n = blockIdx.x * 256 + threadIdx.x; n < N; n += gridDim.x * 256) {
        uint64_t acc = 0;
        for (int k = 0; k < K; k++) {
            const int64_t v = ye[(long)pos[t * K + k] * N + n];
            acc += (uint64_t)((int64_t)((uint64_t)v * (uint64_t)w[t * K + k]) >> shift);
        }
        y[t * N + n] = (int64_t)acc;
    }
}

}  // namespace zk

extern "C" {

void moe_dispatch(const int64_t *indices, int T, int K, int E, int *counts_scratch, int *seg, int *sorted_token,
                  int *sorted_pos, int *tiles, int *ntiles)
{
    const char *name = "moe_dispatch";
    if (T < 0 || K <= 0 || E <= 0) { zk::set_error(zk::kBadArgument, "%s: bad dimension", name); return; }
    if (((!indices || !sorted_token || !sorted_pos) && T > 0) || !counts_scratch || !seg || !tiles || !ntiles) {
        zk::set_error(zk::kBadArgument, "%s: null pointer", name);
        return;
    }
    if (E > 65535) { zk::set_error(zk::kUnsupportedSize, "%s: more than 65535 experts", name); return; }
    const long entries = (long)T * K;
    zk::moe_count_kernel<<<dim3((unsigned)E), dim3(256), 0, 0>>>(indices, entries, counts_scratch);
    zk::moe_scan_kernel<<<dim3(1), dim3(256), 0, 0>>>(counts_scratch, E, seg, tiles, ntiles, entries, sorted_token,
                                                      zk::deferred_error_flag(zk::kDeferredMoeIndex));
    if (entries > 0) zk::moe_place_kernel<<<dim3((unsigned)E), dim3(256), 0, 0>>>(indices, entries, K, seg, sorted_token, sorted_pos);
    zk::check_launch(name);
}

void moe_gather_rows(const int64_t *x, const int *sorted_token, int64_t *out, int rows, int N)
{
    const char *name = "moe_gather_rows";
    if (rows < 0 || N < 0) { zk::set_error(zk::kBadArgument, "%s: negative dimension", name); return; }
    if (rows == 0 || N == 0) return;
    if (!x || !sorted_token || !out) { zk::set_error(zk::kBadArgument, "%s: null pointer", name); return; }
    if (rows > 65535 * 64) { zk::set_error(zk::kUnsupportedSize, "%s: too many rows", name); return; }
    const int vec = N % 2 == 0 && (((uintptr_t)x | (uintptr_t)out) & 15) == 0;
    int bx = (N + 511) / 512;
    if (bx > 16) bx = 16;
    for (long r0 = 0; r0 < rows; r0 += 65535) {
        const long nr = rows - r0 < 65535 ? rows - r0 : 65535;
        zk::moe_gather_kernel<<<dim3((unsigned)bx, (unsigned)nr), dim3(256), 0, 0>>>(x, sorted_token + r0, out + r0 * N, N, vec);
    }
    zk::check_launch(name);
}

void moe_combine(const int64_t *ye, const int64_t *weights, const int *sorted_pos, int64_t *y, int T, int K, int N, int shift)
{
    const char *name = "moe_combine";
    if (T < 0 || K <= 0 || N < 0 || shift < 0 || shift > 63) { zk::set_error(zk::kBadArgument, "%s: bad argument", name); return; }
    if (T == 0 || N == 0) return;
    if (!ye || !weights || !sorted_pos || !y) { zk::set_error(zk::kBadArgument, "%s: null pointer", name); return; }
    int bx = (N + 255) / 256;
    if (bx > 32) bx = 32;
    for (long t0 = 0; t0 < T; t0 += 65535) {
        const long nt = T - t0 < 65535 ? T - t0 : 65535;
        zk::moe_combine_kernel<<<dim3((unsigned)bx, (unsigned)nt), dim3(256), 0, 0>>>(ye, weights + t0 * K, sorted_pos + t0 * K, y + t0 * N, K, N, shift);
    }
    zk::check_launch(name);
}

void int64_grouped_bmm_launcher(const int64_t *A, const void *const *B_ptrs, int b32, int64_t *C, int64_t *R,
                                int64_t c_rescale, const int *seg, const int *tiles, const int *ntiles, int groups,
                                int rows, int K, int N)
{
    const char *name = "int64_grouped_bmm_launcher";
    if (groups < 0 || rows < 0 || K < 0 || N < 0 || c_rescale < 0 || c_rescale > 63) { zk::set_error(zk::kBadArgument, "%s: bad argument", name); return; }
    if (groups == 0 || rows == 0 || N == 0) return;
    if ((!A && K > 0) || !B_ptrs || !C || !seg || !tiles || !ntiles) { zk::set_error(zk::kBadArgument, "%s: null pointer", name); return; }
    zk::GroupedDesc d;
    d.A = A; d.lda = K; d.B = B_ptrs; d.b32 = b32; d.C = C; d.R = R; d.ldc = N;
    d.seg = seg; d.tiles = tiles; d.ntiles = ntiles;
    d.groups = groups; d.rows = rows; d.N = N; d.K = K; d.shift = (int)c_rescale; d.init = 0;
    zk::gemm_grouped_dispatch(name, d);
}

}  // extern "C"
