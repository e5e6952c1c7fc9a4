/*
 * int64gemm.h -- C ABI of libint64gemm.so for AMD MI355X (gfx950).
 *
 * Drop-in replacement for the shared object that the reference builds from
 * inference/int64_gemm.cu and loads with ctypes.CDLL("./libint64gemm.so")
 * (inference/kernel.py:206).  Part 1 declares exactly the entry points that
 * the reference binds, with the same names, argument order, C types and void
 * returns.  Part 2 declares additions that have no counterpart in the
 * reference; nothing in part 1 depends on a caller using them.
 *
 * Conventions shared by every entry point (same as the reference):
 *   - all pointers except the four *_init_* tables are DEVICE pointers owned
 *     by the caller; tensors are contiguous, row-major, little-endian;
 *   - work is enqueued on the null (legacy default) stream and the call
 *     returns without synchronising;
 *   - no return value.  Unlike the reference, argument and launch errors are
 *     recorded and can be read with zk_last_error().
 */
#ifndef ZK_INT64GEMM_H
#define ZK_INT64GEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ======================= Part 1: the reference's ABI ======================= */

/* C[b,m,n] = (sum_k (A[b,m,k]/a_rescale) * (B[n,k]/b_rescale)) >> c_rescale, 128-bit wrapping sum,
 * `/` truncates toward zero; R = sum mod 2^c_rescale.  A [Bdim,M,K] i64, B [N,K], C,R [Bdim,M,N] i64.
 * Replaces inference/int64_gemm.cu:79-90 (B int64) and :36-47 (B int32); bound at inference/kernel.py:209-225.
 * c_rescale must be in [0,63]; the rescales must be non-zero.  R may be NULL (the reference always stores it, but
 * only three of the model's callers read it): then no remainder is stored. */
void int64_64_bmm_broadcast_launcher(const int64_t *A, const int64_t *B, int64_t *C, int64_t *R,
                                     const int64_t a_rescale, const int64_t b_rescale, const int64_t c_rescale,
                                     int Bdim, int M, int K, int N);
void int64_32_bmm_broadcast_launcher(const int64_t *A, const int32_t *B, int64_t *C, int64_t *R,
                                     const int64_t a_rescale, const int64_t b_rescale, const int64_t c_rescale,
                                     int Bdim, int M, int K, int N);

/* RoPE: C = A * B as complex numbers in Q42; every real product is bits [42,106) of the 128-bit product.
 * A,C [batch,seq,heads,headDim,2] i64, B [1,seq,1,headDim,2] i64 (broadcast over batch and heads).
 * Replaces inference/int64_gemm.cu:274-286; bound at inference/kernel.py:227-232. */
void complex_int64_mul(const int64_t *A, const int64_t *B, int64_t *C,
                       int batchSize, int seqLen, int headCount, int headDim);

/* C[s,d] = floor(A[s,d] * W[d] / rms[s]) with a 128-bit product.  A,C [seqLen,Dim] i64, rms [seqLen] i64.
 * Replaces inference/int64_gemm.cu:365-385; bound at inference/kernel.py:234-248. */
void rms_norm_32(const int64_t *A, const int32_t *W, const int64_t *rms, int64_t *C, int seqLen, int Dim);
void rms_norm_64(const int64_t *A, const int64_t *W, const int64_t *rms, int64_t *C, int seqLen, int Dim);

/* MLA einsums, 128-bit accumulation, result (init + sum) >> rescale with init = rescale/2 (half the shift
 * COUNT) for the first three and 0 for the last.  Replace inference/int64_gemm.cu:416-425, :458-467,
 * :499-509, :539-549; bound at inference/kernel.py:250-280.
 *   bshd,hdc->bshc : A [B,S,H,D] i64,  W [H,D,C] i32,   out [B,S,H,C]
 *   bshc,btc->bsht : A [B,S,H,C] i64,  Bm [B,T,C] i64,  out [B,S,H,T]
 *   bsht,btc->bshc : A [B,S,H,T] i64,  Bm [B,T,C] i64,  out [B,S,H,C]
 *   bshc,hdc->bshd : A [B,S,H,C] i64,  W [H,D,C] i32,   out [B,S,H,D]                                   */
void einsum_bshd_hdc_bshc(const int64_t *q_nope, const int32_t *wkv_b_1, int64_t *out,
                          int64_t rescale, int B, int S, int H, int D, int C);
void einsum_bshc_btc_bsht(const int64_t *A, const int64_t *B, int64_t *C,
                          int64_t rescale, int Bsz, int S, int H, int T, int Cdim);
void einsum_bsht_btc_bshc(const int64_t *A, const int64_t *B, int64_t *C,
                          int64_t rescale, int Bsz, int S, int H, int T, int Cdim);
void einsum_bshc_hdc_bshd(const int64_t *A, const int32_t *B, int64_t *C,
                          int64_t rescale, int Bsz, int S, int H, int D, int Cdim);

/* Fixed-point softmax over the last dim of R [Bsz,S,H,T] i64 into C; LUT = 256 x i64 on the device.
 * Replace inference/int64_gemm.cu:661-670 (Q21, rounded divide) and :748-757 (Q19, truncating divide);
 * bound at inference/kernel.py:282-294.  The reference leaves the per-element weights in R; this
 * library leaves R untouched unless zk_softmax_clobber_input(1) was called. */
void softmax_q21(int64_t *R, int64_t *C, int64_t *EXP2_FRAC_LUT, int Bsz, int S, int H, int T);
void softmax_q19(int64_t *R, int64_t *C, int64_t *EXP2_FRAC_LUT, int Bsz, int S, int H, int T);

/* Fill a HOST table of 256 i64.  Replace inference/int64_gemm.cu:672-680, :759-767, :832-839, :960-967;
 * bound at inference/kernel.py:296-302, 318-320, 336-338. */
void softmax_init_q21(int64_t *EXP2_FRAC_LUT);
void softmax_init_q19(int64_t *EXP2_FRAC_LUT);
void silu_init_q25(int64_t *EXP2_FRAC_LUT);
void silu_init_q23(int64_t *EXP2_FRAC_LUT);

/* Elementwise SiLU / sigmoid over R [Bsz,S,Dim] i64 into C.  Replace inference/int64_gemm.cu:821-830,
 * :884-893, :949-958, :1019-1028; bound at inference/kernel.py:304-334. */
void silu_q25(int64_t *R, int64_t *C, int64_t *EXP2_FRAC_LUT_25, int Bsz, int S, int Dim);
void sigmoid_q25(int64_t *R, int64_t *C, int64_t *EXP2_FRAC_LUT_25, int Bsz, int S, int Dim);
void silu_q23(int64_t *R, int64_t *C, int64_t *EXP2_FRAC_LUT_23, int Bsz, int S, int Dim);
void sigmoid_q23(int64_t *R, int64_t *C, int64_t *EXP2_FRAC_LUT_23, int Bsz, int S, int Dim);

/* Exported by the reference but bound by none of its Python (inference/int64_gemm.cu:126-132, :173-179,
 * :215-221): bit-level bf16 / fp32 -> fixed-point conversion of a [rows,cols] matrix. */
void bf16_to_int32_2d(const uint16_t *input, int32_t *output, int rows, int cols, int rescale);
void wkv_b_bf16_to_int32(const uint16_t *input, int32_t *output, int rows, int cols);
void float32_to_int64_2d(const uint32_t *input, int64_t *output, int rows, int cols, int rescale);

/* ================= Part 2: additions (no reference counterpart) ============ */

/* Error channel.  0 = no error since the last zk_clear_error().  Codes: 1 bad argument, 2 launch failure,
 * 3 unsupported size. */
int zk_last_error(void);
const char *zk_last_error_string(void);
void zk_clear_error(void);

/* The reference's library allocates nothing and keeps no state; this one keeps scratch buffers on the device between
 * calls (digit planes of A, partial sums of split tiles, range slots, a row-major copy of a small B, the quotient
 * tables of the activations), allocated on demand and grown inside a call when a larger problem arrives.
 * zk_workspace_bytes: device bytes held as scratch right now.  zk_prepared_weights_bytes: device bytes held as digit
 * planes made by zk_gemm_prepare_weights.  zk_release_workspace: waits for the device and frees the scratch (not the
 * prepared weights: zk_gemm_release_weights returns those); later calls allocate again what they need. */
size_t zk_workspace_bytes(void);
size_t zk_prepared_weights_bytes(void);
void zk_release_workspace(void);
/* Reads the diagnosis switches ZK_GEMM_SYNC, ZK_NO_TAIL_SPLIT, ZK_B_ROWS_MIN_MACS, ZK_ROWS16_MAX_WEIGHTS and ZK_SKINNY_MAX_M from the
 * environment again (they are read once when the library is loaded, not per call). */
void zk_reload_env(void);

/* RMS statistic on the device: rms[m] = isqrt((eps + sum_n A[m,n]^2) / dim), exact (192-bit sum).
 * Replaces the host loop of inference/kernel.py:477-494 and :539-542 (one .item() sync per element). */
void rms_stat_int64(const int64_t *A, int64_t *rms, int M, int N, int64_t eps, int64_t dim);

/* Statistic and normalisation in one launch (the row is read from HBM once); rms [M] is also written. */
void rms_norm_fused_32(const int64_t *A, const int32_t *W, int64_t *rms, int64_t *C,
                       int M, int N, int64_t eps, int64_t dim);
void rms_norm_fused_64(const int64_t *A, const int64_t *W, int64_t *rms, int64_t *C,
                       int M, int N, int64_t eps, int64_t dim);

/* The residual connection fused into the norm behind it: X' = X + Y * 2^k (wrapping int64, as the tensor ops of
 * inference/model.py:1465 and :1472 compute it) is stored to Xout [M,N] (which may be X itself) and normalised in
 * the same pass over the row: C = floor(X' * W / rms), rms as above.  32 bytes per element instead of the 56 of
 * multiply, add and norm as three tensor ops.  0 <= k <= 63. */
void rms_norm_residual_fused_32(const int64_t *X, const int64_t *Y, int k, const int32_t *W, int64_t *Xout, int64_t *rms,
                                int64_t *C, int M, int N, int64_t eps, int64_t dim);
void rms_norm_residual_fused_64(const int64_t *X, const int64_t *Y, int k, const int64_t *W, int64_t *Xout, int64_t *rms,
                                int64_t *C, int M, int N, int64_t eps, int64_t dim);

/* 1: softmax_q19/q21 also overwrite R with the per-element weights, as the reference's kernels do
 * (inference/int64_gemm.cu:708,729 and :629,650).  0 (default): R is left untouched. */
void zk_softmax_clobber_input(int on);

/* Fusion around the softmax (no counterpart in the reference's library; it replaces the tensor ops of
 * inference/model.py:896-906 and the softmax_q19 call of :908-915 by one pass):
 *   x = floor((s1 + s2) * mul / div) + mask[s][t];   scores = x (if not null);   C = softmax_q19(x)
 * s1, s2 (may be null), scores (may be null), C: [Bsz,S,H,T]; mask (may be null): [S,T] broadcast over batch and
 * heads; 0 < div < 2^31; arithmetic wraps like torch's int64 ops; the floor division is torch's `//`.
 * Rows longer than 2048 need the scores buffer. */
void softmax_q19_scores(const int64_t *s1, const int64_t *s2, const int64_t *mask, int64_t *scores, int64_t *C,
                        const int64_t *lut, int Bsz, int S, int H, int T, int64_t mul, int64_t div);

/* Fusion around the SiLU of the FFNs (no counterpart in the reference's library; it replaces silu_q23 plus the
 * tensor ops of inference/model.py:1039-1048 and :1271-1280):  C = (silu_q23(R) * U) >> 23 with a wrapping product;
 * the SiLU values themselves are stored to S when S is not null.  All tensors [Bsz,S,Dim]. */
void silu_mul_q23(const int64_t *R, const int64_t *U, int64_t *S, int64_t *C, const int64_t *lut, int Bsz, int Sq, int Dim);

/* Expert routing of the MoE gate (no counterpart in the reference's library; it replaces the tensor ops of
 * Gate.forward, inference/model.py:1143-1208, on the output of sigmoid_q23).  scores [T,E] int64 (Q23), bias [E]
 * int32 or null.  Per token: biased scores; each of the n_groups groups scored by the sum of its two largest biased
 * scores (its maximum without bias); the topk_groups best groups kept, the others count as -2^42; the topk largest
 * biased scores win, in descending order, ties to the lower index (torch.topk leaves ties to its implementation).
 * indices [T,topk] int64; raw_weights [T,topk] (may be null) = the winners' UNBIASED scores (gate_weights.bin);
 * weights [T,topk] = floor(floor(raw * 2^23 / sum raw) * 5 / 2).  E <= 1024, n_groups <= 64 dividing E, topk <= 64. */
void gate_route_q23(const int64_t *scores, const int32_t *bias, int64_t *weights, int64_t *indices,
                    int64_t *raw_weights, int T, int E, int n_groups, int topk_groups, int topk);

/* The same routing straight from the gate's logits (no counterpart in the reference's library; it replaces sigmoid_q23
 * plus the tensor ops of inference/model.py:1135-1208 by one launch): every logit goes through sigmoid_q23 (table `lut`,
 * 256 entries as the silu/sigmoid kernels take it) first.  scores [T,E] (may be null) receives the sigmoid values, i.e.
 * what gate_route_q23 takes as input and the reference dumps as sigmoid_gate_y.bin / gate_original_scores.bin. */
void gate_sigmoid_route_q23(const int64_t *logits, const int64_t *lut, const int32_t *bias, int64_t *scores,
                            int64_t *weights, int64_t *indices, int64_t *raw_weights, int T, int E, int n_groups,
                            int topk_groups, int topk);

/* Witness dump writer (replaces the reference's saveTensor, inference/model.py:94-102: a synchronous .cpu() copy and
 * file write per tensor, ~30 per layer).  zk_dump_device queues the raw bytes of `bytes` bytes of contiguous device
 * memory for `path`: the copy to pinned host memory is ordered on the null stream behind the kernels that produced
 * the data and ahead of anything launched later, so the caller may overwrite or free the tensor right after the call
 * returns; a writer thread writes the file (created or truncated) once the copy has landed.  zk_dump_host does the
 * same for host memory (copied before it returns).  Both return 0, or -1 with zk_last_error set.  Files are complete
 * only after zk_dump_flush(), which waits for everything queued and returns the number of dumps that failed. */
int zk_dump_device(const char *path, const void *device_ptr, size_t bytes);
int zk_dump_host(const char *path, const void *host_ptr, size_t bytes);
long zk_dump_flush(void);

/* MoE dispatch on the device (no counterpart in the reference's library; together these replace the Python loop over
 * the experts of MoE.forward, inference/model.py:1325-1383).  All pointers are device pointers.
 *
 * moe_dispatch: indices [T,K] int64 (expert of every routed (token, slot) entry, as gate_route_q23 returns them) ->
 *   seg [E+1]: first row of every expert's segment in the sorted order (seg[E] = T*K);
 *   sorted_token [T*K]: the token of every sorted row (tokens ascending within an expert, as torch.where gives them);
 *   sorted_pos [T*K]: the sorted row of entry (t, k);
 *   tiles [2 * (T*K/32 + E)], ntiles [1]: the 32-row tiles of the segments, for int64_grouped_bmm_launcher;
 *   counts_scratch [E]: scratch.
 *   An index outside [0, E) belongs to no segment: seg[E] < T*K then, the entry's sorted_pos is 0 (moe_combine reads
 *   row 0 for it), the unowned rows behind seg[E] get token 0, and the error is recorded once the kernels have run
 *   (zk_last_error after a synchronisation, or any later call's check); nothing reads outside the buffers.
 * moe_gather_rows: out[r][:] = x[sorted_token[r]][:]  (x [T,N], out [rows,N]).
 * int64_grouped_bmm_launcher: C[r][n] = (sum_k A[r][k] * B_e[n][k]) >> c_rescale (128-bit wrapping sum) and, when R
 *   is not null, R = that sum mod 2^c_rescale, for the rows r of expert e's segment; B_ptrs [groups] holds the
 *   experts' weight matrices ([N,K], int32 when b32 else int64).  Semantics of int64_64/32_bmm_broadcast_launcher
 *   per segment.  The first call with a table of weights waits for the device once (its digit check); later calls
 *   with that table do not wait: like the bmm launchers they run on remembered digit counts and are followed by a
 *   guarded recomputation (see zk_gemm_guard_hits).
 * moe_combine: y[t][n] = sum_k (ye[sorted_pos[t][k]][n] * weights[t][k]) >> shift with wrapping products and sums
 *   (model.py:1379 with shift 23; floor, like torch's //). */
void moe_dispatch(const int64_t *indices, int T, int K, int E, int *counts_scratch, int *seg, int *sorted_token,
                  int *sorted_pos, int *tiles, int *ntiles);
void moe_gather_rows(const int64_t *x, const int *sorted_token, int64_t *out, int rows, int N);
void int64_grouped_bmm_launcher(const int64_t *A, const void *const *B_ptrs, int b32, int64_t *C, int64_t *R,
                                int64_t c_rescale, const int *seg, const int *tiles, const int *ntiles, int groups,
                                int rows, int K, int N);
void moe_combine(const int64_t *ye, const int64_t *weights, const int *sorted_pos, int64_t *y, int T, int K, int N, int shift);

/* No counterpart in the reference.  For callers that cannot allocate device memory (tight serving loops,
 * harnesses that forbid hipMalloc; NOT for capture into a HIP graph as it stands: its two kernels are launched on the
 * null stream, which a capturing stream does not record, and the first call on a device also looks up the array's
 * address and sets a kernel attribute): the product of int64_64/32_bmm_broadcast_launcher (b32 != 0: B
 * holds int32) for up to 16 rows, a_rescale fixed at 1 and b_rescale a positive power of two, on kernels whose scratch
 * (the partial sums of a K split) is a static 8 MB array in device memory instead of a buffer the library allocates.
 * It allocates nothing, frees nothing and waits for nothing.  Limits: M <= 16 and Bdim * M * N <= 2^20 outputs; anything
 * beyond is rejected with error 3.  Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two
 * streams, two threads) race.  Nothing in the array needs clearing: a call writes every slot it reads.  Same bits as the
 * existing entry points; R may be NULL. */
void int64_bmm_broadcast_noalloc(const int64_t *A, const void *B, int b32, int64_t *C, int64_t *R,
                                 int64_t b_rescale, int64_t c_rescale, int Bdim, int M, int K, int N);

/* GEMM instruction path for the bmm launchers and the einsums: 0 = automatic (default),
 * 1 = native VALU 64-bit multiply-add chains, 2 = limb-decomposed i8 MFMA.  Results are identical. */
void zk_gemm_set_path(int path);
int zk_gemm_get_path(void);
/* What the last GEMM-like call used: path (1/2) and the limb counts of A and B (0 for the VALU path, and for the
 * MFMA kernels for up to 16 rows, which take their digit counts from the data step by step). */
void zk_gemm_last_plan(int *path, int *limbs_a, int *limbs_b);
/* i8 digit products per int64 multiply-add in the last GEMM-like call (0 for the VALU path).  At most
 * limbs_a * limbs_b; fewer when the stored bits [shift, shift + 64) of the sum lie below the weight of the top
 * digit pairs, which are then not multiplied at all. */
int zk_gemm_last_pairs(void);
/* The MFMA path guesses how many base-256 digits the operands need (from what the same pointers, or the last operands
 * of the same shape, needed) and checks the guess on the device.  No call waits for that check: a guarded launch
 * behind it (the widest MFMA instance, or the vector-ALU tiles where that does not apply) recomputes the outputs if the
 * guess was too small.  This returns how many calls so far needed that recomputation (counted once their ranges have
 * reached the host; it waits for nothing). */
long zk_gemm_guard_hits(void);
/* How many int64_grouped_bmm_launcher calls so far ran as ONE launch over all groups (the others went group by group). */
long zk_gemm_grouped_mfma_calls(void);
/* How many of those launches ran on the kernel that streams int32 weights through LDS rings (K a multiple of 32,
 * sixteen digit pairs or more; ZK_STREAM32_MIN_PAIRS and ZK_NO_STREAM32 move or remove that choice). */
long zk_gemm_grouped_streamed_calls(void);
/* How many GEMM launches so far ran on the software-pipelined 128 x 128 kernel that reads digit planes on both sides
 * (weights prepared with zk_gemm_prepare_weights, three digits a side; ZK_NO_PIPE=1 switches it off). */
long zk_gemm_pipe_calls(void);
/* No reference counterpart: model weights do not change between calls, so a weight matrix W[N,K] (int64, or int32 with
 * b32 != 0; groups == 0, B = the device pointer later passed as B) or all the matrices of a device table of pointers
 * (groups > 0, B = the table later passed to int64_grouped_bmm_launcher) can be split into base-256 digit planes ONCE.
 * Later calls of int64_64/32_bmm_broadcast_launcher / int64_grouped_bmm_launcher with that pointer, these N and K,
 * b_rescale 1 and contiguous rows then read the planes (as many bytes per weight as its values need digits: 3 for
 * |w| < 2^23, 4 up to 31 bits, else 5 or 9) and split nothing of B; results are the same bits.  The library allocates
 * the planes and keeps them until zk_gemm_release_weights or the end of the process.  The original weights must stay
 * where they are and unchanged meanwhile (the exact fallback path and the matrix-vector kernels read them).  The planes
 * are found by ADDRESS and nothing of B is read or range-checked on that path: if the weights are freed without
 * zk_gemm_release_weights and an allocator hands the address to another matrix of the same shape, that matrix is
 * multiplied with the old planes and the results are silently wrong.  Release before freeing (the Python wrapper keeps
 * the tensor alive until release_weights).  Returns 0 on success; an error is recorded otherwise.  Waits for the device. */
int zk_gemm_prepare_weights(const void *B, int b32, int groups, int N, int K);
void zk_gemm_release_weights(const void *B);
/* 1 when the last GEMM-like call ran on the MFMA path and read B from prepared planes, else 0. */
int zk_gemm_last_prepared(void);

/* Measurement helper for the roofline of the MFMA GEMM path: the sustained rate, in 10^12 i8 operations per
 * second (2 per multiply-add), of a stream of v_mfma_i32_32x32x32_i8 shaped like the GEMM's inner loop (8 waves
 * per compute unit, 10 accumulator tiles per wave).  with_lds: operand fragments re-read from LDS and a
 * barrier per step, as in the GEMM; otherwise register resident.  random_data: operands are random bytes
 * instead of zeros (the device is power managed and the rate depends on how the operand bits toggle).
 * Allocates 4 bytes for the duration of the call and waits for its kernels. */
double zk_probe_mfma_i8_tops(int with_lds, int random_data, int steps);
/* Microseconds per repetition of two dependent, nearly empty launches back to back on the null stream (`workgroups`
 * workgroups store 16 bytes each, a second kernel reads them): what the launches alone cost a call that is made of a
 * streaming kernel and a finishing kernel.  A measurement aid for bench.py; not needed for inference. */
double zk_probe_launch_pair_us(int workgroups, int reps);
/* GB/s of non-temporal 16-byte stores into a buffer of `bytes` bytes with nothing read: what the device takes in writes
 * alone, the ceiling of the write-heavy converters.  A measurement aid for bench.py. */
double zk_probe_store_gbps(long bytes, int reps);

/* HIP-event stopwatch on the null stream (the stream every entry point launches on). */
void zk_timer_start(void);
float zk_timer_stop_ms(void);   /* records the stop event, waits for it, returns elapsed milliseconds */

/* Float checkpoint -> fixed-point weights, the quantisation of inference/convert2.py on the device.
 * fp8_block_scaled_to_int32: out = (weight_dequant(w, scale).to(float32) * 2^k).round().to(int32)
 * (convert2.py:144-147, 308-311 and the like; weight_dequant is the Triton kernel of inference/kernel.py:67-117):
 * w [rows,cols] OCP e4m3fn bytes, scale [ceil(rows/128), ceil(cols/128)] float32, one scale per 128x128 block; the
 * product is rounded to bfloat16 (the reference's default dtype, convert2.py:185) before it is scaled by 2^k, rounded
 * half to even and converted as the reference's device converts (saturating, NaN -> 0).  0 <= k <= 127.
 * bf16_scaled_round_to_int32/64: out = (p.to(float32) * 2^k).round().to(int32|int64) for n bfloat16 values
 * (convert2.py:250-262, 290-295, 353-359). */
void fp8_block_scaled_to_int32(const uint8_t *w, const float *scale, int32_t *out, int rows, int cols, int k);
void bf16_scaled_round_to_int32(const uint16_t *in, int32_t *out, long n, int k);
void bf16_scaled_round_to_int64(const uint16_t *in, int64_t *out, long n, int k);

#ifdef __cplusplus
}
#endif
#endif /* ZK_INT64GEMM_H */
