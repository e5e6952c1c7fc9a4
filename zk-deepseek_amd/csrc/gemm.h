// One descriptor for every GEMM-shaped entry point (the two bmm launchers and the four MLA einsums):
//
//   C[g][m][n] = (init + sum_k (A[g][m][k] / a_rs) * (B[g][n,k] / b_rs)) >> shift      (128-bit wrapping sum)
//   R[g][m][n] = (that sum) mod 2^shift                                                 (optional)
//
// A is always k-contiguous.  B is either k-contiguous ("n-major", ldbk == 1: weights [N,K], K^T of the
// attention scores) or n-contiguous ("k-major", ldbn == 1: V of P.V, wkv_b_1 [D,C]).
#pragma once
#include "common.h"

namespace zk {

struct GemmDesc {
    const int64_t *A;
    long lda, sA;             // A[g][m][k] = A[g * sA + m * lda + k]
    const void *B;
    int b32;                  // 1: B holds int32, 0: int64
    long ldbn, ldbk, sB;      // B[g][n,k] = B[g * sB + n * ldbn + k * ldbk]; exactly one of ldbn, ldbk is 1
    int64_t *C, *R;           // R may be null
    long ldc, sC;             // C[g][m][n] = C[g * sC + m * ldc + n]
    int G, M, N, K;
    int shift;                // 0..63
    int64_t init;             // added to the sum before the shift
    int64_t a_rs, b_rs;       // operand divisors (truncating), 1 = none
};

enum GemmPath { kPathAuto = 0, kPathValu = 1, kPathMfma = 2 };

// Native 64-bit multiply-add chains on the vector ALU; handles every descriptor.  With a `guard` (device
// pointer) the launch is conditional: its workgroups return at once unless *guard is non-zero when they start.
void gemm_valu_launch(const GemmDesc &d, const unsigned long long *guard = nullptr);

// Matrix-vector kernel of the same family for one or two rows of A against k-contiguous B: one launch, nothing
// guessed.  Returns false (nothing launched) for any other descriptor.
bool gemm_gemv_launch(const GemmDesc &d);

// Limb-decomposed i8 MFMA.  Returns 0 when the product was launched, 1 when the descriptor is outside what it
// supports or memory for its buffers is short (nothing was launched; the caller falls back to the VALU path), -1 on an
// error (recorded).  The outcome describes this call only, whatever the sticky error channel holds from earlier ones.
int gemm_mfma_launch(const GemmDesc &d, int *limbs_a, int *limbs_b);

// A handful of rows (M <= 16) against k-contiguous B on the 16-row MFMA tiles: every wavefront on its own, digit counts
// taken from the data (nothing guessed, nothing read back), K split over wavefronts when the launch would not fill the
// device otherwise (a second, small launch then adds the slices' partial sums).  acc: scratch for those sums (`max_slots`
// slots of 8 KB: one per output tile of 16 x 32 and workgroup of slices; nothing in it needs clearing); null: the library's
// own, grown on demand.  Returns 0 when launched, 1 when the descriptor is outside what it takes (nothing launched), -1
// on an error (recorded).
int gemm_rows16_launch(const GemmDesc &d, unsigned long long *acc = nullptr, size_t max_slots = 0);
size_t gemm_rows16_workspace_bytes();
void gemm_rows16_release_workspace();
void gemm_rows16_reload_switches();

// Calls of the MFMA path that returned before their verdict was known and turned out to need the guarded
// vector-ALU recomputation (known once their range has reached the host).
long gemm_mfma_guard_hits();
// weights prepared once as digit planes (an int64 or int32 matrix, or a device table of `groups` of them): 0 on success
int gemm_mfma_prepare(const void *B, int b32, int groups, int N, int K);
void gemm_mfma_release(const void *B);
bool gemm_mfma_is_prepared(const void *B);
int gemm_mfma_last_pairs();       // digit pairs multiplied per element of K by the last MFMA launch
int gemm_mfma_last_prepared();    // 1 when the last MFMA launch read B from prepared planes
long gemm_mfma_grouped_streamed_calls();   // grouped launches so far that ran on the streamed int32 kernel
long gemm_mfma_pipe_calls();               // launches so far that ran on the software-pipelined kernel for planes on both sides

// Grouped product: the rows of A and C form one contiguous segment per group and every group has its own
// k-contiguous B[N,K] (the experts of a MoE layer after the tokens have been sorted by expert):
//   C[r][n] = (init + sum_k A[r][k] * B_group(r)[n][k]) >> shift,   R likewise.
// Everything that describes the segments lives on the device, so the host never learns the segment sizes.
struct GroupedDesc {
    const int64_t *A;
    long lda;
    const void *const *B;     // device array of `groups` device pointers
    int b32;
    int64_t *C, *R;           // R may be null
    long ldc;
    const int *seg;           // device [groups + 1]: first row of every segment, seg[groups] = rows
    const int *tiles;         // device [2 * (rows / 32 + groups)]: {group, first row} of every 32-row tile
    const int *ntiles;        // device [1]: how many of those tiles exist
    int groups, rows, N, K, shift;
    int64_t init;
};

// The grouped product row by row on the matrix-vector kernel: one launch, every row of A against the B of its segment.
// Streams a B once per row of its segment, so it is for a handful of rows (a decoding step's routed experts).
// Returns false (nothing launched) when the descriptor is outside what it takes.
bool gemm_gemv_grouped_launch(const GroupedDesc &d);

// The grouped product on the 16-row MFMA tiles (see gemm_rows16_launch): one launch, no wait.  0 / 1 / -1 as there.
// `guard`: a device word; when given, the launch's workgroups return at once unless it is non-zero (the fallback behind
// a speculative launch of the 32-row kernels).
int gemm_rows16_grouped(const GroupedDesc &d, const unsigned long long *guard = nullptr);

// One launch of the 32-row-tile MFMA kernels over all groups.  Returns 0 when done, 1 when the operands need
// more digits than those kernels are built for (nothing valid was written: the caller takes another route),
// -1 on an error (recorded).
int gemm_mfma_grouped(const GroupedDesc &d, int *limbs_a, int *limbs_b);

// Grouped product through the MFMA launch above or, where that does not apply (path forced to VALU, K = 0,
// operands wider than its kernels take), group by group through gemm_dispatch after one read-back of the segments.
void gemm_grouped_dispatch(const char *name, const GroupedDesc &d);

// Top-level dispatch used by the extern "C" launchers.  False when this call failed (the error is recorded).
bool gemm_dispatch(const char *name, const GemmDesc &d);

}  // namespace zk
