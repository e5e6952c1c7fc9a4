/*
 * zk_oracle.c -- TEST INFRASTRUCTURE ONLY.
 *
 * Scalar CPU restatement (plain C, __int128) of the int64 fixed-point
 * arithmetic that the reference's libint64gemm.so computes on the GPU.
 * It is the checker for the HIP library: only tests/, __graft_entry__.smoke()
 * and bench.py's cpu_baseline leg may load it.  The product never calls it.
 *
 * Every function cites the reference lines it follows
 * (paths relative to the reference repository root).
 *
 * Semantics that the reference leaves to the hardware are fixed here and are
 * marked "parity unpinned" (nothing in the reference can confirm them):
 *   - GEMM remainder R for c_rescale >= 32 (reference builds its mask in a
 *     32-bit int, inference/int64_gemm.cu:22,65): here R = sum mod 2^c.
 *   - SiLU/sigmoid `t << k` for k >= 40 (signed overflow) and k >= 64
 *     (inference/int64_gemm.cu:812,878,940,1008): here the shift is done on
 *     the unsigned pattern and yields 0 for k >= 64 (NVIDIA's clamped shift).
 *   - softmax q21 with x - max wrapping past 2^63 (k < 0): t >> 63.
 *   - division by zero (rms == 0, 2^23 + u == 0): result 0.
 *   - INT64_MIN / -1: wraps to INT64_MIN.
 * Everything else is pinned by tests/test_oracle_*.py.
 */
#include <stdint.h>
#include <stddef.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef __int128 i128;
typedef unsigned __int128 u128;

static int g_threads = 1;

void ora_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int ora_get_threads(void) { return g_threads; }
int ora_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* C++ `/` on int64 (truncation toward zero) with the two UB corners fixed. */
static inline int64_t tdiv64(int64_t a, int64_t b)
{
    if (b == 0) return 0;
    if (b == -1) return (int64_t)(0 - (uint64_t)a);
    return a / b;
}

static inline int64_t shr128_to64(u128 sum, int c)
{
    /* arithmetic shift of the signed 128-bit pattern, then truncation */
    return (int64_t)(uint64_t)((i128)sum >> c);
}

/* ------------------------------------------------------------------------
 * Generic strided GEMM core shared by the bmm launchers and the einsums:
 *   out[g][m][n] = (init + sum_k A[g][m][k] * B[g][n,k]) >> shift
 * B element (n,k) lives at  B + g*sB + n*ldbn + k*ldbk  (int32 or int64).
 * ---------------------------------------------------------------------- */
static void gemm_core(const int64_t *A, long lda, long sA,
                      const void *B, int b32, long ldbn, long ldbk, long sB,
                      int64_t *C, int64_t *R, long ldc, long sC,
                      int G, int M, int N, int K,
                      int64_t a_rs, int64_t b_rs, int shift, int64_t init)
{
    long total = (long)G * M;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (long gm = 0; gm < total; gm++) {
        int g = (int)(gm / M), m = (int)(gm % M);
        const int64_t *a = A + (long)g * sA + (long)m * lda;
        for (int n = 0; n < N; n++) {
            u128 sum = (u128)(i128)init;
            if (b32) {
                const int32_t *b = (const int32_t *)B + (long)g * sB + (long)n * ldbn;
                if (a_rs == 1 && b_rs == 1) {
                    for (int k = 0; k < K; k++)
                        sum += (u128)((i128)a[k] * (i128)b[(long)k * ldbk]);
                } else {
                    for (int k = 0; k < K; k++)
                        sum += (u128)((i128)tdiv64(a[k], a_rs) *
                                      (i128)tdiv64((int64_t)b[(long)k * ldbk], b_rs));
                }
            } else {
                const int64_t *b = (const int64_t *)B + (long)g * sB + (long)n * ldbn;
                if (a_rs == 1 && b_rs == 1) {
                    for (int k = 0; k < K; k++)
                        sum += (u128)((i128)a[k] * (i128)b[(long)k * ldbk]);
                } else {
                    for (int k = 0; k < K; k++)
                        sum += (u128)((i128)tdiv64(a[k], a_rs) *
                                      (i128)tdiv64(b[(long)k * ldbk], b_rs));
                }
            }
            long o = (long)g * sC + (long)m * ldc + n;
            C[o] = shr128_to64(sum, shift);
            if (R) {
                uint64_t lo = (uint64_t)sum;
                R[o] = (int64_t)(shift == 0 ? 0 : (shift >= 64 ? lo : (lo & ((1ULL << shift) - 1))));
            }
        }
    }
}

/* inference/int64_gemm.cu:49-90 (kernel + launcher), W int64.
 * sum += int128(a / a_rescale) * int128(b / b_rescale)   (:69)
 * C = int64(sum >> c_rescale)  (:74),  R = int64(sum & ((1<<c)-1))  (:65,:75) */
void ora_int64_64_bmm_broadcast(const int64_t *A, const int64_t *B, int64_t *C, int64_t *R,
                                int64_t a_rs, int64_t b_rs, int64_t c_rs,
                                int Bdim, int M, int K, int N)
{
    gemm_core(A, K, (long)M * K, B, 0, K, 1, 0, C, R, N, (long)M * N,
              Bdim, M, N, K, a_rs, b_rs, (int)c_rs, 0);
}

/* inference/int64_gemm.cu:6-47, W int32 (b_val / b_rescale is done in int64, :26). */
void ora_int64_32_bmm_broadcast(const int64_t *A, const int32_t *B, int64_t *C, int64_t *R,
                                int64_t a_rs, int64_t b_rs, int64_t c_rs,
                                int Bdim, int M, int K, int N)
{
    gemm_core(A, K, (long)M * K, B, 1, K, 1, 0, C, R, N, (long)M * N,
              Bdim, M, N, K, a_rs, b_rs, (int)c_rs, 0);
}

/* inference/int64_gemm.cu:387-425.  out[b,s,h,c] = (rescale/2 + sum_d q[b,s,h,d]*W[h,d,c]) >> rescale,
 * W int32 [H,D,C]; note the rounding term is half the SHIFT COUNT (:401). */
void ora_einsum_bshd_hdc_bshc(const int64_t *A, const int32_t *W, int64_t *out,
                              int64_t rescale, int B, int S, int H, int D, int C)
{
    /* batch = head; rows = (b,s) with row stride H*D (in) and H*C (out) */
    for (int h = 0; h < H; h++)
        gemm_core(A + (long)h * D, (long)H * D, 0,
                  W + (long)h * D * C, 1, 1, C, 0,
                  out + (long)h * C, NULL, (long)H * C, 0,
                  1, B * S, C, D, 1, 1, (int)rescale, rescale / 2);
}

/* inference/int64_gemm.cu:427-467.  out[b,s,h,t] = (rescale/2 + sum_c A[b,s,h,c]*Bm[b,t,c]) >> rescale (:442-452). */
void ora_einsum_bshc_btc_bsht(const int64_t *A, const int64_t *Bm, int64_t *out,
                              int64_t rescale, int Bsz, int S, int H, int T, int Cdim)
{
    gemm_core(A, Cdim, (long)S * H * Cdim,
              Bm, 0, Cdim, 1, (long)T * Cdim,
              out, NULL, T, (long)S * H * T,
              Bsz, S * H, T, Cdim, 1, 1, (int)rescale, rescale / 2);
}

/* inference/int64_gemm.cu:469-509.  out[b,s,h,c] = (rescale/2 + sum_t P[b,s,h,t]*V[b,t,c]) >> rescale (:483-493). */
void ora_einsum_bsht_btc_bshc(const int64_t *A, const int64_t *V, int64_t *out,
                              int64_t rescale, int Bsz, int S, int H, int T, int Cdim)
{
    gemm_core(A, T, (long)S * H * T,
              V, 0, 1, Cdim, (long)T * Cdim,
              out, NULL, Cdim, (long)S * H * Cdim,
              Bsz, S * H, Cdim, T, 1, 1, (int)rescale, rescale / 2);
}

/* inference/int64_gemm.cu:511-549.  out[b,s,h,d] = (sum_c A[b,s,h,c]*W[h,d,c]) >> rescale, init 0 (:525), W int32. */
void ora_einsum_bshc_hdc_bshd(const int64_t *A, const int32_t *W, int64_t *out,
                              int64_t rescale, int Bsz, int S, int H, int D, int Cdim)
{
    for (int h = 0; h < H; h++)
        gemm_core(A + (long)h * Cdim, (long)H * Cdim, 0,
                  W + (long)h * D * Cdim, 1, Cdim, 1, 0,
                  out + (long)h * D, NULL, (long)H * D, 0,
                  1, Bsz * S, D, Cdim, 1, 1, (int)rescale, 0);
}

/* inference/int64_gemm.cu:223-286.  p(a,b) = bits [42,106) of the signed 128-bit product (:257-260);
 * re = p(a0,b0) - p(a1,b1), im = p(a0,b1) + p(a1,b0) (:262-263); B index = s*headDim + d (:245). */
static inline int64_t mul_q42(int64_t a, int64_t b)
{
    return (int64_t)(uint64_t)(((i128)a * (i128)b) >> 42);
}

void ora_complex_int64_mul(const int64_t *A, const int64_t *Bt, int64_t *C,
                           int batch, int seq, int heads, int headDim)
{
    long total = (long)batch * seq * heads * headDim;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (long idx = 0; idx < total; idx++) {
        long i = idx;
        int d = (int)(i % headDim); i /= headDim;
        i /= heads;
        int s = (int)(i % seq);
        long bi = (long)s * headDim + d;
        int64_t a0 = A[2 * idx], a1 = A[2 * idx + 1];
        int64_t b0 = Bt[2 * bi], b1 = Bt[2 * bi + 1];
        C[2 * idx]     = (int64_t)((uint64_t)mul_q42(a0, b0) - (uint64_t)mul_q42(a1, b1));
        C[2 * idx + 1] = (int64_t)((uint64_t)mul_q42(a0, b1) + (uint64_t)mul_q42(a1, b0));
    }
}

/* inference/kernel.py:477-494 (int64_RMS0): rms = isqrt((eps + sum a^2) // dim) in unbounded ints.
 * sum a^2 can reach 2^139, so the accumulator is 192 bits (three 64-bit words). */
typedef struct { uint64_t w[3]; } u192;

static inline void u192_add128(u192 *x, u128 v)
{
    u128 t = (u128)x->w[0] + (uint64_t)v;
    x->w[0] = (uint64_t)t;
    t = (u128)x->w[1] + (uint64_t)(v >> 64) + (uint64_t)(t >> 64);
    x->w[1] = (uint64_t)t;
    x->w[2] += (uint64_t)(t >> 64);
}

/* floor(x / d) for 0 < d < 2^63, by long division on 64-bit words */
static inline u192 u192_div64(u192 x, uint64_t d)
{
    u192 q;
    u128 rem = 0;
    for (int i = 2; i >= 0; i--) {
        u128 cur = (rem << 64) | x.w[i];
        q.w[i] = (uint64_t)(cur / d);
        rem = cur % d;
    }
    return q;
}

/* floor(sqrt(x)) for x < 2^128 */
static uint64_t isqrt128(u128 x)
{
    if (x == 0) return 0;
    /* bit-by-bit restoring square root: exact, no floating point */
    u128 res = 0, bit = (u128)1 << 126;
    while (bit > x) bit >>= 2;
    while (bit != 0) {
        if (x >= res + bit) { x -= res + bit; res = (res >> 1) + bit; }
        else res >>= 1;
        bit >>= 2;
    }
    return (uint64_t)res;
}

/* rms[m] for each row of A [M,N].  Returns -1 if (eps+sum)//dim needs more than 128 bits
 * (cannot happen for dim >= 2^11, never at the model's shapes). */
int ora_rms_stat(const int64_t *A, int64_t *rms, int M, int N, int64_t eps, int64_t dim)
{
    int bad = 0;
    for (int m = 0; m < M; m++) {
        u192 acc = { { 0, 0, 0 } };
        u192_add128(&acc, (u128)(i128)eps);   /* eps >= 0 in every caller (model.py:486-493 passes 1) */
        for (int n = 0; n < N; n++) {
            int64_t a = A[(long)m * N + n];
            u192_add128(&acc, (u128)((i128)a * (i128)a));
        }
        u192 q = u192_div64(acc, (uint64_t)dim);
        if (q.w[2] != 0) { bad = -1; rms[m] = 0; continue; }
        rms[m] = (int64_t)isqrt128(((u128)q.w[1] << 64) | q.w[0]);
    }
    return bad;
}

/* inference/int64_gemm.cu:289-385.  prod = int128(a)*int128(w); qq = prod / r; rr = prod % r;
 * if (rr < 0) qq -= 1; C = int64(qq)  (:314-324, :352-362). */
static inline int64_t rms_apply(int64_t a, int64_t w, int64_t r)
{
    if (r == 0) return 0;
    i128 prod = (i128)a * (i128)w;
    i128 qq = prod / (i128)r;
    i128 rr = prod % (i128)r;
    if (rr < 0) qq -= 1;
    return (int64_t)(uint64_t)(u128)qq;
}

void ora_rms_norm_32(const int64_t *A, const int32_t *W, const int64_t *rms, int64_t *C, int seqLen, int Dim)
{
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int s = 0; s < seqLen; s++)
        for (int d = 0; d < Dim; d++)
            C[(long)s * Dim + d] = rms_apply(A[(long)s * Dim + d], (int64_t)W[d], rms[s]);
}

void ora_rms_norm_64(const int64_t *A, const int64_t *W, const int64_t *rms, int64_t *C, int seqLen, int Dim)
{
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int s = 0; s < seqLen; s++)
        for (int d = 0; d < Dim; d++)
            C[(long)s * Dim + d] = rms_apply(A[(long)s * Dim + d], W[d], rms[s]);
}

/* ---- LUT initialisers: host functions in the reference too ------------- */
/* inference/int64_gemm.cu:759-767: LUT[i] = int64(pow(2, i*(-1.0f)/256) * 2^19) */
void ora_softmax_init_q19(int64_t *lut)
{
    for (int i = 0; i < 256; i++) lut[i] = (int64_t)(pow(2.0, (double)(i * (-1.0f) / 256)) * (double)(1 << 19));
}
/* inference/int64_gemm.cu:672-680 */
void ora_softmax_init_q21(int64_t *lut)
{
    for (int i = 0; i < 256; i++) lut[i] = (int64_t)(pow(2.0, (double)(i * (-1.0f) / 256)) * (double)(1 << 21));
}
/* inference/int64_gemm.cu:960-967: LUT[i] = int64(pow(2, i*1.0f/256) * 2^23) */
void ora_silu_init_q23(int64_t *lut)
{
    for (int i = 0; i < 256; i++) lut[i] = (int64_t)(pow(2.0, (double)(i * 1.0f / 256)) * 8388608.0);
}
/* inference/int64_gemm.cu:832-839 */
void ora_silu_init_q25(int64_t *lut)
{
    for (int i = 0; i < 256; i++) lut[i] = (int64_t)(pow(2.0, (double)(i * 1.0f / 256)) * 33554432.0);
}

/* ---- softmax ------------------------------------------------------------ */
static inline int64_t sar_clamped(int64_t t, int64_t k)
{
    if (k < 0 || k > 63) return t >> 63;
    return t >> k;
}

/* inference/int64_gemm.cu:684-746.  Rows are the last dim of [B,S,H,T].
 * W (optional) receives the per-element weights w that the reference writes back into R (:708,:729). */
void ora_softmax_q19(const int64_t *Rin, int64_t *C, int64_t *W, const int64_t *lut,
                     int Bsz, int S, int H, int T)
{
    long rows = (long)Bsz * S * H;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (long r = 0; r < rows; r++) {
        const int64_t *x = Rin + r * T;
        int64_t *c = C + r * T;
        int64_t rmax = x[0];
        for (int i = 1; i < T; i++) if (x[i] > rmax) rmax = x[i];
        uint64_t sumW = 0;
        for (int i = 0; i < T; i++) {
            uint64_t d = (uint64_t)rmax - (uint64_t)x[i];          /* :703 */
            int64_t wi;
            if (d > ((uint64_t)64 << 19)) wi = 0;                  /* :706 */
            else {
                int64_t y = (int64_t)(((u128)d * (u128)756388) >> 19);   /* :713 */
                int64_t k = y >> 19;                               /* :715 */
                int64_t f = y & 0x7FFFF;                           /* :716 */
                int64_t t = lut[f >> 11];                          /* :720 */
                wi = (k >= 64) ? 0 : (t >> k);                     /* :723 */
            }
            c[i] = wi;            /* staged in the output row, replaced below */
            sumW += (uint64_t)wi;
        }
        int64_t s = (int64_t)sumW;
        for (int i = 0; i < T; i++) {
            int64_t wi = c[i];
            if (W) W[r * T + i] = wi;
            int64_t num = (int64_t)((uint64_t)wi << 19);           /* :739 */
            c[i] = s ? tdiv64(num, s) : 0;                         /* :740 */
        }
    }
}

/* inference/int64_gemm.cu:605-659 */
void ora_softmax_q21(const int64_t *Rin, int64_t *C, int64_t *W, const int64_t *lut,
                     int Bsz, int S, int H, int T)
{
    long rows = (long)Bsz * S * H;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (long r = 0; r < rows; r++) {
        const int64_t *x = Rin + r * T;
        int64_t *c = C + r * T;
        int64_t rmax = x[0];
        for (int i = 1; i < T; i++) if (x[i] > rmax) rmax = x[i];
        uint64_t sumW = 0;
        for (int i = 0; i < T; i++) {
            int64_t d = (int64_t)((uint64_t)x[i] - (uint64_t)rmax);     /* :624 */
            int64_t wi;
            if (d < -((int64_t)64 << 21)) wi = 0;                       /* :627 */
            else {
                int64_t y = (int64_t)((uint64_t)d * 3025551ULL + (1ULL << 20)) >> 21;   /* :634 */
                int64_t ny = (int64_t)(0 - (uint64_t)y);
                int64_t k = ny >> 21;                                   /* :636 */
                int64_t f = ny & 0x1FFFFF;                              /* :637 */
                int64_t t = lut[f >> 13];                               /* :641 */
                wi = (k >= 64) ? 0 : sar_clamped(t, k);                 /* :644 */
            }
            c[i] = wi;
            sumW += (uint64_t)wi;
        }
        int64_t s = (int64_t)sumW;
        for (int i = 0; i < T; i++) {
            int64_t wi = c[i];
            if (W) W[r * T + i] = wi;
            int64_t num = (int64_t)((uint64_t)wi << 21);                /* :656 */
            c[i] = s ? tdiv64((int64_t)((uint64_t)num + (uint64_t)(s / 2)), s) : 0;   /* :657 */
        }
    }
}

/* ---- SiLU / sigmoid ----------------------------------------------------- */
static inline int64_t exp2_fixed(int64_t y, int Q, const int64_t *lut)
{
    /* u = 2^(y / 2^Q) in Q-bit fixed point: inference/int64_gemm.cu:935-940 (q23), :807-812 (q25) */
    int64_t k = y >> Q;
    int64_t f = y & (((int64_t)1 << Q) - 1);
    int64_t t = lut[f >> (Q - 8)];
    int64_t u = 0;
    if (k > -63) {
        if (k < 0) u = t >> (-k);
        else u = (k >= 64) ? 0 : (int64_t)((uint64_t)t << k);
    }
    return u;
}

static inline int64_t recip_fixed(int64_t u, int Q)
{
    int64_t den = (int64_t)(((uint64_t)1 << Q) + (uint64_t)u);
    return tdiv64((int64_t)1 << (2 * Q), den);
}

/* mode 0 = SiLU, 1 = sigmoid.  q23: inference/int64_gemm.cu:903-947, :969-1017.
 * Both return r unchanged for r >= 2^29 (sigmoid too, :986-991) and 0 for r <= -2^29. */
void ora_act_q23(const int64_t *Rin, int64_t *C, const int64_t *lut, long n, int mode)
{
    const int64_t LIM = (int64_t)64 << 23;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (long i = 0; i < n; i++) {
        int64_t r = Rin[i];
        if (r >= LIM) { C[i] = r; continue; }
        if (r <= -LIM) { C[i] = 0; continue; }
        int64_t y = (int64_t)(uint64_t)(((i128)(-r) * (i128)12102203) >> 23);   /* :932 negate BEFORE the shift */
        int64_t q = recip_fixed(exp2_fixed(y, 23, lut), 23);                    /* :943 */
        C[i] = mode ? q : (int64_t)((uint64_t)r * (uint64_t)q) >> 23;           /* :946 / :1016 */
    }
}

/* q25: inference/int64_gemm.cu:775-819, :841-882.  y = -int64((r*LOG2E)>>25): negate AFTER the shift (:804). */
void ora_act_q25(const int64_t *Rin, int64_t *C, const int64_t *lut, long n, int mode)
{
    const int64_t LIM = (int64_t)64 << 25;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (long i = 0; i < n; i++) {
        int64_t r = Rin[i];
        if (r >= LIM) { C[i] = r; continue; }
        if (r <= -LIM) { C[i] = 0; continue; }
        int64_t y = -(int64_t)(uint64_t)(((i128)r * (i128)48408813) >> 25);
        int64_t q = recip_fixed(exp2_fixed(y, 25, lut), 25);
        C[i] = mode ? q : (int64_t)((uint64_t)r * (uint64_t)q) >> 25;
    }
}

/* ---- float bit patterns -> fixed point (exported by the reference, bound by none of its Python) ---------
 * inference/int64_gemm.cu:92-132 (bf16 -> int32), :134-179 (wkv_b variant: 2^25 scale, saturates |x| >= 0.5),
 * :181-221 (fp32 -> int64).  value = (1.mantissa) * 2^(exp + rescale), truncated toward zero, sign applied last.
 * The reference forms `1 << ex2` in 32-bit int: shifts of 32 or more are hardware-defined there; here a left
 * shift of 32 or more multiplies by 0 and a right shift of 31 or more divides to 0 (parity unpinned). */
static uint32_t scale_mantissa_u32(uint32_t r2, int ex2)
{
    if (ex2 >= 0) return ex2 >= 32 ? 0u : r2 * (1u << ex2);
    return -ex2 >= 31 ? 0u : r2 / (1u << -ex2);
}

void ora_bf16_to_int32(const uint16_t *in, int32_t *out, long n, int rescale, int wkv_b)
{
    for (long i = 0; i < n; i++) {
        int v0 = in[i];
        int ex0 = ((v0 >> 7) & 0xFF) - 127;
        int r0 = v0 & 0x7F;
        if (ex0 == -127 && r0 == 0) { out[i] = 0; continue; }                 /* :104-107 */
        if (wkv_b && ex0 >= -1) { out[i] = 0x7FFFFFFF; continue; }            /* :151-154 */
        uint32_t v = scale_mantissa_u32((uint32_t)(r0 + 128), ex0 + rescale); /* :109-116 */
        if (v0 & 0x8000) v = 0u - v;                                          /* :118-120 */
        out[i] = (int32_t)v;
    }
}

void ora_float32_to_int64(const uint32_t *in, int64_t *out, long n, int rescale)
{
    for (long i = 0; i < n; i++) {
        uint32_t v0 = in[i];
        int ex0 = (int)((v0 >> 23) & 0xFF) - 127;
        int r0 = (int)(v0 & 0x7FFFFF);
        if (ex0 == -127 && r0 == 0) { out[i] = 0; continue; }
        int ex2 = ex0 + rescale;
        int64_t r2 = (int64_t)r0 + 8388608;
        int64_t v;
        if (ex2 >= 0) v = ex2 >= 32 ? 0 : (int64_t)((uint64_t)r2 * (uint64_t)(int64_t)(int32_t)(1u << ex2));   /* :202 */
        else v = -ex2 >= 31 ? 0 : r2 / (int64_t)(1u << -ex2);                                                   /* :204 */
        if (v0 & 0x80000000u) v = (int64_t)(0 - (uint64_t)v);
        out[i] = v;
    }
}

/* ---- expert routing of the MoE gate ------------------------------------------------------------
 * The tensor ops of Gate.forward after sigmoid_q23 (inference/model.py:1143-1208), per token:
 *   s = scores + bias (:1149); group score = sum of the two largest s of the group (:1166), the maximum when
 *   there is no bias (:1162); the topk_groups best groups are kept (:1172), every s of the others becomes -2^42
 *   (:1185); indices = the topk largest s (:1189); raw = scores gathered at indices (:1194);
 *   weights = (raw * 2^23) // sum(raw) (:1203), then * 5 // 2 (:1208), `//` being floor division.
 * torch.topk returns its winners in descending order and leaves ties to its implementation: here the lower
 * index wins (parity unpinned on ties; sigmoid scores plus a bias rarely tie).  sum(raw) == 0 gives 0. */
static int64_t ora_floordiv(int64_t a, int64_t b)
{
    if (b == 0) return 0;
    int64_t q = a / b;
    if ((a % b != 0) && ((a < 0) != (b < 0))) q--;
    return q;
}

void ora_gate_route(const int64_t *scores, const int32_t *bias, int64_t *weights, int64_t *indices, int64_t *raw,
                    int T, int E, int n_groups, int topk_groups, int topk)
{
    const int64_t masked = -((int64_t)1 << 42);
#pragma omp parallel for schedule(static) num_threads(g_threads)
    for (int t = 0; t < T; t++) {
        int64_t s[1024];
        char gone[1024], keep[64], used[64];
        int64_t gs[64];
        const int64_t *row = scores + (long)t * E;
        for (int e = 0; e < E; e++) s[e] = (int64_t)((uint64_t)row[e] + (uint64_t)(int64_t)(bias ? bias[e] : 0));
        if (n_groups > 1) {
            const int gsize = E / n_groups;
            for (int g = 0; g < n_groups; g++) {
                int i1 = -1, i2 = -1;
                for (int e = g * gsize; e < (g + 1) * gsize; e++)
                    if (i1 < 0 || s[e] > s[i1]) i1 = e;
                for (int e = g * gsize; e < (g + 1) * gsize; e++)
                    if (e != i1 && (i2 < 0 || s[e] > s[i2])) i2 = e;
                gs[g] = bias ? (int64_t)((uint64_t)s[i1] + (uint64_t)(i2 >= 0 ? s[i2] : 0)) : s[i1];
                keep[g] = 0;
                used[g] = 0;
            }
            for (int k = 0; k < topk_groups; k++) {
                int best = -1;
                for (int g = 0; g < n_groups; g++)
                    if (!used[g] && (best < 0 || gs[g] > gs[best])) best = g;
                used[best] = 1;
                keep[best] = 1;
            }
            for (int e = 0; e < E; e++)
                if (!keep[e / gsize]) s[e] = masked;
        }
        for (int e = 0; e < E; e++) gone[e] = 0;
        int64_t sum = 0;
        for (int k = 0; k < topk; k++) {
            int best = -1;
            for (int e = 0; e < E; e++)
                if (!gone[e] && (best < 0 || s[e] > s[best])) best = e;
            gone[best] = 1;
            indices[(long)t * topk + k] = best;
            weights[(long)t * topk + k] = row[best];
            sum = (int64_t)((uint64_t)sum + (uint64_t)row[best]);
        }
        for (int k = 0; k < topk; k++) {
            int64_t w = weights[(long)t * topk + k];
            if (raw) raw[(long)t * topk + k] = w;
            w = ora_floordiv((int64_t)((uint64_t)w << 23), sum);
            weights[(long)t * topk + k] = ora_floordiv((int64_t)((uint64_t)w * 5u), 2);
        }
    }
}
