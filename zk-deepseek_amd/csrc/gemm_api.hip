// extern "C" launchers of the GEMM-shaped entry points: argument checks, descriptor construction and the
// choice between the VALU and the MFMA instruction path.
#include "gemm.h"
#include "../../include/int64gemm.h"

#include <vector>

namespace zk {

static int g_gemm_path = kPathAuto;
static int g_last_path = 0, g_last_la = 0, g_last_lb = 0;
static bool g_last_digits = false;      // the last call ran on kernels with fixed digit counts (gemm_mfma.hip), whose plan and planes are reported
static long g_grouped_mfma_calls = 0;

// An empty contraction (K == 0): every output is the rounding term shifted, as the reference's loop over no elements leaves
// it (int64_gemm.cu:44-78); A and B hold nothing and are never read.
static __global__ void gemm_empty_k_kernel(int64_t *C, int64_t *R, long ldc, long sC, int M, int N, long total, int64_t quotient, int64_t remainder)
{
    for (long o = (long)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (long)gridDim.x * blockDim.x) {
        const long g = o / ((long)M * N), r = o - g * ((long)M * N);
        const long at = g * sC + (r / N) * ldc + r % N;
        C[at] = quotient;
        if (R) R[at] = remainder;
    }
}

static bool gemm_empty_k(const char *name, int64_t *C, int64_t *R, long ldc, long sC, int G, int M, int N, int shift, int64_t init)
{
    const long total = (long)G * M * N;
    if (total == 0) return true;
    const int64_t mask = shift ? (int64_t)(((uint64_t)1 << shift) - 1) : 0;
    const long blocks = (total + 255) / 256;
    gemm_empty_k_kernel<<<dim3((unsigned)(blocks < 4096 ? blocks : 4096)), 256, 0, 0>>>(C, R, ldc, sC, M, N, total, init >> shift, init & mask);
    g_last_path = kPathValu; g_last_la = 0; g_last_lb = 0; g_last_digits = false;
    return check_launch(name);
}

bool gemm_dispatch(const char *name, const GemmDesc &d)
{
    if (d.K == 0) return gemm_empty_k(name, d.C, d.R, d.ldc, d.sC, d.G, d.M, d.N, d.shift, d.init);
    // one or two rows (a decoding step, the head): the exact vector-ALU stream over the weights, unless the MFMA
    // path is asked for by name
    // (prepared weights: the MFMA kernels read a few bytes per weight where the matrix-vector stream reads eight, so
    // from 128 MB of weights on they go first and the matrix-vector kernels only if the MFMA path does not take the
    // product.  One row against [18432,7168]: 0.19 -> 0.087 ms; against [576,7168] the stream wins, 9 against 22 us.)
    const bool prepared = g_gemm_path != kPathValu && !d.b32 && (long)d.N * d.K >= (16L << 20) && gemm_mfma_is_prepared(d.B);
    if (g_gemm_path != kPathMfma && !prepared && gemm_gemv_launch(d)) {
        g_last_path = kPathValu; g_last_la = 0; g_last_lb = 0; g_last_digits = false;
        return check_launch(name);
    }
    // up to 16 rows against k-contiguous weights: the 16-row MFMA tiles, digit counts taken from the data on the device
    // (prepared weights keep the kernels that read their planes: fewer bytes per weight)
    if (g_gemm_path != kPathValu && !gemm_mfma_is_prepared(d.B)) {
        const int rc = gemm_rows16_launch(d);
        if (rc == 0) {
            g_last_path = kPathMfma; g_last_la = 0; g_last_lb = 0; g_last_digits = false;
            return check_launch(name);
        }
        if (rc < 0) return false;
    }
    if (g_gemm_path != kPathValu) {
        int la = 0, lb = 0;
        // 0: launched, 1: declined (whatever the error channel holds comes from an earlier call and must not keep this
        // one from running on the other path), -1: failed and recorded
        const int rc = gemm_mfma_launch(d, &la, &lb);
        if (rc == 0) {
            g_last_path = kPathMfma; g_last_la = la; g_last_lb = lb; g_last_digits = true;
            return check_launch(name);
        }
        if (rc < 0) return false;
    }
    if (g_gemm_path != kPathMfma && prepared && gemm_gemv_launch(d)) {
        g_last_path = kPathValu; g_last_la = 0; g_last_lb = 0; g_last_digits = false;
        return check_launch(name);
    }
    gemm_valu_launch(d);
    g_last_path = kPathValu; g_last_la = 0; g_last_lb = 0; g_last_digits = false;
    return check_launch(name);
}

// rows up to which the grouped product is offered to the matrix-vector kernels, which go row by row (a few tokens at
// top-8).  Measured on config 5's experts with int32 weights: 8 rows 0.27 ms against 0.95 ms on the 32-row MFMA kernels,
// 64 rows 1.85 against 2.18 ms, 128 rows 3.4 against 3.3 ms.  (The launcher itself stops at 32 rows for products that
// its LDS-staged kernel does not take.)
constexpr int kGroupedGemvMaxRows = 64;

void gemm_grouped_dispatch(const char *name, const GroupedDesc &d)
{
    if (d.K == 0) { gemm_empty_k(name, d.C, d.R, d.ldc, 0, 1, d.rows, d.N, d.shift, d.init); return; }
    // (prepared weights: from 33 rows on the MFMA kernels first, as in gemm_dispatch; below that the handful of tiles
    // leaves most of the device idle and the row-by-row stream is faster: one token 0.52 against 0.66 ms)
    const bool prepared = g_gemm_path != kPathValu && !d.b32 && d.rows > 32 && gemm_mfma_is_prepared((const void *)d.B);
    const bool few_rows = g_gemm_path != kPathMfma && d.rows <= kGroupedGemvMaxRows && d.K > 0;
    if (few_rows && !prepared && gemm_gemv_grouped_launch(d)) {
        g_last_path = kPathValu; g_last_la = 0; g_last_lb = 0; g_last_digits = false;
        check_launch(name);
        return;
    }
    if (g_gemm_path != kPathValu && d.K > 0) {
        int la = 0, lb = 0;
        const int rc = gemm_mfma_grouped(d, &la, &lb);
        if (rc == 0) {
            g_last_path = kPathMfma; g_last_la = la; g_last_lb = lb; g_last_digits = true;
            g_grouped_mfma_calls++;
            check_launch(name);
            return;
        }
        if (rc < 0) return;
    }
    // operands wider than the 32-row kernels take (or K == 0): the 16-row tiles, which take their digit counts from
    // the data and recompute on the vector ALU what is wider still.  One launch as well, and no wait.  (On the experts'
    // usual widths the 32-row kernels stream faster: 4.9 against 2.4 TB/s of int32 weights.)
    if (g_gemm_path != kPathValu) {
        const int rc = gemm_rows16_grouped(d);
        if (rc == 0) {
            g_last_path = kPathMfma; g_last_la = 0; g_last_lb = 0; g_last_digits = false;
            g_grouped_mfma_calls++;
            check_launch(name);
            return;
        }
        if (rc < 0) return;
    }
    if (few_rows && prepared && gemm_gemv_grouped_launch(d)) {
        g_last_path = kPathValu; g_last_la = 0; g_last_lb = 0; g_last_digits = false;
        check_launch(name);
        return;
    }
    // group by group: the segment table and the B pointers come to the host once
    std::vector<int> seg((size_t)d.groups + 1);
    std::vector<const void *> bp((size_t)d.groups);
    if (hipMemcpy(seg.data(), d.seg, seg.size() * sizeof(int), hipMemcpyDeviceToHost) != hipSuccess ||
        hipMemcpy(bp.data(), d.B, bp.size() * sizeof(void *), hipMemcpyDeviceToHost) != hipSuccess) {
        set_error(kLaunchFailure, "%s: cannot read the segment table", name);
        return;
    }
    for (int e = 0; e < d.groups; e++) {
        const int r0 = seg[e], m = seg[e + 1] - seg[e];
        if (m <= 0) continue;
        GemmDesc g;
        g.A = d.A + (long)r0 * d.lda; g.lda = d.lda; g.sA = 0;
        g.B = bp[e]; g.b32 = d.b32; g.ldbn = d.K; g.ldbk = 1; g.sB = 0;
        g.C = d.C + (long)r0 * d.ldc; g.R = d.R ? d.R + (long)r0 * d.ldc : nullptr; g.ldc = d.ldc; g.sC = 0;
        g.G = 1; g.M = m; g.N = d.N; g.K = d.K;
        g.shift = d.shift; g.init = d.init; g.a_rs = 1; g.b_rs = 1;
        if (!gemm_dispatch(name, g)) return;
    }
}

static bool dims_ok(const char *name, std::initializer_list<int> dims, int64_t shift)
{
    for (int v : dims)
        if (v < 0) { set_error(kBadArgument, "%s: negative dimension", name); return false; }
    if (shift < 0 || shift > 63) {
        set_error(kBadArgument, "%s: shift %lld outside [0,63]", name, (long long)shift);
        return false;
    }
    return true;
}

static void bmm(const char *name, const int64_t *A, const void *B, int b32, int64_t *C, int64_t *R,
                int64_t a_rs, int64_t b_rs, int64_t c_rs, int Bdim, int M, int K, int N)
{
    if (!dims_ok(name, { Bdim, M, K, N }, c_rs)) return;
    if (a_rs == 0 || b_rs == 0) { set_error(kBadArgument, "%s: zero rescale divisor", name); return; }
    if ((long)Bdim * M * N == 0) return;
    if (((!A || !B) && K > 0) || !C) { set_error(kBadArgument, "%s: null pointer", name); return; }
    GemmDesc d;
    d.A = A; d.lda = K; d.sA = (long)M * K;
    d.B = B; d.b32 = b32; d.ldbn = K; d.ldbk = 1; d.sB = 0;
    d.C = C; d.R = R; d.ldc = N; d.sC = (long)M * N;
    d.G = Bdim; d.M = M; d.N = N; d.K = K;
    d.shift = (int)c_rs; d.init = 0; d.a_rs = a_rs; d.b_rs = b_rs;
    gemm_dispatch(name, d);
}

}  // namespace zk

extern "C" {

void int64_64_bmm_broadcast_launcher(const int64_t *A, const int64_t *B, int64_t *C, int64_t *R,
                                     const int64_t a_rescale, const int64_t b_rescale, const int64_t c_rescale,
                                     int Bdim, int M, int K, int N)
{
    zk::bmm("int64_64_bmm_broadcast_launcher", A, B, 0, C, R, a_rescale, b_rescale, c_rescale, Bdim, M, K, N);
}

void int64_32_bmm_broadcast_launcher(const int64_t *A, const int32_t *B, int64_t *C, int64_t *R,
                                     const int64_t a_rescale, const int64_t b_rescale, const int64_t c_rescale,
                                     int Bdim, int M, int K, int N)
{
    zk::bmm("int64_32_bmm_broadcast_launcher", A, B, 1, C, R, a_rescale, b_rescale, c_rescale, Bdim, M, K, N);
}

// out[b,s,h,c] = (rescale/2 + sum_d q[b,s,h,d] * W[h,d,c]) >> rescale: one GEMM per head, rows (b,s).
void einsum_bshd_hdc_bshc(const int64_t *q_nope, const int32_t *wkv_b_1, int64_t *out, int64_t rescale,
                          int B, int S, int H, int D, int C)
{
    const char *name = "einsum_bshd_hdc_bshc";
    if (!zk::dims_ok(name, { B, S, H, D, C }, rescale)) return;
    if ((long)B * S * H * C == 0) return;
    if (((!q_nope || !wkv_b_1) && D > 0) || !out) { zk::set_error(zk::kBadArgument, "%s: null pointer", name); return; }
    zk::GemmDesc d;
    d.A = q_nope; d.lda = (long)H * D; d.sA = D;
    d.B = wkv_b_1; d.b32 = 1; d.ldbn = 1; d.ldbk = C; d.sB = (long)D * C;
    d.C = out; d.R = nullptr; d.ldc = (long)H * C; d.sC = C;
    d.G = H; d.M = B * S; d.N = C; d.K = D;
    d.shift = (int)rescale; d.init = rescale / 2; d.a_rs = 1; d.b_rs = 1;
    zk::gemm_dispatch(name, d);
}

// out[b,s,h,t] = (rescale/2 + sum_c A[b,s,h,c] * Bm[b,t,c]) >> rescale: one GEMM per batch, rows (s,h).
void einsum_bshc_btc_bsht(const int64_t *A, const int64_t *B, int64_t *C, int64_t rescale,
                          int Bsz, int S, int H, int T, int Cdim)
{
    const char *name = "einsum_bshc_btc_bsht";
    if (!zk::dims_ok(name, { Bsz, S, H, T, Cdim }, rescale)) return;
    if ((long)Bsz * S * H * T == 0) return;
    if (((!A || !B) && Cdim > 0) || !C) { zk::set_error(zk::kBadArgument, "%s: null pointer", name); return; }
    zk::GemmDesc d;
    d.A = A; d.lda = Cdim; d.sA = (long)S * H * Cdim;
    d.B = B; d.b32 = 0; d.ldbn = Cdim; d.ldbk = 1; d.sB = (long)T * Cdim;
    d.C = C; d.R = nullptr; d.ldc = T; d.sC = (long)S * H * T;
    d.G = Bsz; d.M = S * H; d.N = T; d.K = Cdim;
    d.shift = (int)rescale; d.init = rescale / 2; d.a_rs = 1; d.b_rs = 1;
    zk::gemm_dispatch(name, d);
}

// out[b,s,h,c] = (rescale/2 + sum_t P[b,s,h,t] * V[b,t,c]) >> rescale: one GEMM per batch, V is k-major.
void einsum_bsht_btc_bshc(const int64_t *A, const int64_t *B, int64_t *C, int64_t rescale,
                          int Bsz, int S, int H, int T, int Cdim)
{
    const char *name = "einsum_bsht_btc_bshc";
    if (!zk::dims_ok(name, { Bsz, S, H, T, Cdim }, rescale)) return;
    if ((long)Bsz * S * H * Cdim == 0) return;
    if (((!A || !B) && T > 0) || !C) { zk::set_error(zk::kBadArgument, "%s: null pointer", name); return; }
    zk::GemmDesc d;
    d.A = A; d.lda = T; d.sA = (long)S * H * T;
    d.B = B; d.b32 = 0; d.ldbn = 1; d.ldbk = Cdim; d.sB = (long)T * Cdim;
    d.C = C; d.R = nullptr; d.ldc = Cdim; d.sC = (long)S * H * Cdim;
    d.G = Bsz; d.M = S * H; d.N = Cdim; d.K = T;
    d.shift = (int)rescale; d.init = rescale / 2; d.a_rs = 1; d.b_rs = 1;
    zk::gemm_dispatch(name, d);
}

// out[b,s,h,d] = (sum_c A[b,s,h,c] * W[h,d,c]) >> rescale (no rounding term): one GEMM per head.
void einsum_bshc_hdc_bshd(const int64_t *A, const int32_t *B, int64_t *C, int64_t rescale,
                          int Bsz, int S, int H, int D, int Cdim)
{
    const char *name = "einsum_bshc_hdc_bshd";
    if (!zk::dims_ok(name, { Bsz, S, H, D, Cdim }, rescale)) return;
    if ((long)Bsz * S * H * D == 0) return;
    if (((!A || !B) && Cdim > 0) || !C) { zk::set_error(zk::kBadArgument, "%s: null pointer", name); return; }
    zk::GemmDesc d;
    d.A = A; d.lda = (long)H * Cdim; d.sA = Cdim;
    d.B = B; d.b32 = 1; d.ldbn = Cdim; d.ldbk = 1; d.sB = (long)D * Cdim;
    d.C = C; d.R = nullptr; d.ldc = (long)H * D; d.sC = D;
    d.G = H; d.M = Bsz * S; d.N = D; d.K = Cdim;
    d.shift = (int)rescale; d.init = 0; d.a_rs = 1; d.b_rs = 1;
    zk::gemm_dispatch(name, d);
}

void zk_gemm_set_path(int path)
{
    if (path < 0 || path > 2) { zk::set_error(zk::kBadArgument, "zk_gemm_set_path: path %d outside [0,2]", path); return; }
    zk::g_gemm_path = path;
}

int zk_gemm_get_path(void) { return zk::g_gemm_path; }

void zk_gemm_last_plan(int *path, int *limbs_a, int *limbs_b)
{
    if (path) *path = zk::g_last_path;
    if (limbs_a) *limbs_a = zk::g_last_la;
    if (limbs_b) *limbs_b = zk::g_last_lb;
}

long zk_gemm_guard_hits(void) { return zk::gemm_mfma_guard_hits(); }
int zk_gemm_last_pairs(void) { return zk::g_last_digits ? zk::gemm_mfma_last_pairs() : 0; }

long zk_gemm_grouped_mfma_calls(void) { return zk::g_grouped_mfma_calls; }
long zk_gemm_grouped_streamed_calls(void) { return zk::gemm_mfma_grouped_streamed_calls(); }
long zk_gemm_pipe_calls(void) { return zk::gemm_mfma_pipe_calls(); }

int zk_gemm_last_prepared(void) { return zk::g_last_digits ? zk::gemm_mfma_last_prepared() : 0; }
int zk_gemm_prepare_weights(const void *B, int b32, int groups, int N, int K) { return zk::gemm_mfma_prepare(B, b32, groups, N, K); }
void zk_gemm_release_weights(const void *B) { zk::gemm_mfma_release(B); }

}  // extern "C"
