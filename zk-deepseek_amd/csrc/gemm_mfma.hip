// GEMM path (b): limb-decomposed i8 MFMA.
//
// Every int64 operand x is written in balanced base-256 digits, x = sum_j d_j * 256^j with d_j in [-128,127].
// The digits come from one 64-bit add and one xor: with bias_n = 0x80 in bytes 0..n-2,
//     d_j = byte_j(x + bias_n) - 128  (j < n-1),   d_{n-1} = signed byte_{n-1}(x + bias_n),
// which is exact whenever x + bias_n fits n signed bytes; n = 9 covers all of int64 (d_8 in {0,1}).
// The product sum then splits into digit-pair GEMMs that run on v_mfma_i32_32x32x32_i8,
//     sum_k a*b = sum_{i,j} 256^(i+j) * (sum_k da_i * db_j),
// all pairs with the same i+j share one int32 accumulator tile, and the epilogue recombines the
// NA+NB-1 diagonals with carries into the 128-bit sum before the shift.  Nothing is approximated.
//
// Operand tiles are converted on the fly: a thread gathers 8 elements of one row, splits them into digits with
// v_perm_b32 byte transposes and stores each digit plane to LDS already in MFMA fragment order (lane l of a
// fragment = row l%32, k-half l/32, 16 bytes), so the inner loop is ds_read_b128 + MFMA.
// A dot product does not care about the order of k as long as both operands use the same one, so the 8
// elements a thread owns are NOT consecutive: thread j of a row owns runs of RUN consecutive k spaced
// RUN*OCTS apart.  Adjacent lanes then read adjacent 16-byte pieces and every 64-byte line of the tile is
// fetched by exactly one load instruction.
//
// The digit counts are speculated from a cached or sampled range.  The kernels track the exact min and max of
// everything they load (every workgroup leaves its share in a slot of its own, a few workgroups fold
// them and compare with the digit counts used).  The first call for an operand reads the verdict back and
// reruns with wider digits if the guess was too small.  Later calls do not wait: a guarded launch of the
// vector-ALU kernel follows, which recomputes everything if the verdict is bad and returns at once otherwise,
// and the exact range travels to the host behind the stream to refresh the cache.  Results never depend on
// the guess, and a call whose operands were seen before never blocks the host.
#include "gemm_mfma_kernels.h"

#include <map>
#include <mutex>
#include <set>
#include <tuple>

namespace zk {

// the 128 x 128 kernel for digit planes on both sides (gemm_mfma_pipe.h), by digit counts (or null), and its dynamic LDS
MfmaKernel pipe_kernel(int na, int nb);
size_t pipe_lds_size(int na, int nb);

// the streamed form of the grouped launch for int32 weights (gemm_stream32.h), by digit counts; null: none
MfmaKernel stream32_grouped_kernel(int na, int nb, size_t *lds);
MfmaKernel stream32_grouped_kernel_wide(int na, int nb, size_t *lds);

// Digit-count combinations that are compiled.  A request is rounded up to the cheapest one that covers it.
static const Instance *instances(int *count)
{
    static const std::vector<Instance> table = [] {
        std::vector<Instance> t;
#ifdef ZK_PROBE
        const Instance probe[] = { ZK_PROBE };
        t.assign(probe, probe + sizeof(probe) / sizeof(probe[0]));
#else
        mfma_instances_narrow(t);
        mfma_instances_mid(t);
        mfma_instances_wide(t);
        mfma_instances_pruned(t);
        mfma_instances_rows32(t);
        mfma_instances_rows32b(t);
        mfma_instances_rows32c(t);
        mfma_instances_rows32d(t);
        mfma_instances_rows32e(t);
#endif
        return t;
    }();
    *count = (int)table.size();
    return table.data();
}

// need_diag: the result's top bit is below 2^(8 need_diag), so diagonals from need_diag up cannot reach it
// exact_nb / variant: for B from prepared planes the instance must have exactly the planes' digit count and that kernel
static const Instance *pick_instance(int na, int nb, bool b32, bool skinny, int need_diag = 16, int exact_nb = 0, int variant = -1, int exact_kk = 1)
{
    int count;
    const Instance *t = instances(&count);
    const Instance *best = nullptr;
    long best_cost = 0;
    for (int i = 0; i < count; i++) {
        if (t[i].na < na || t[i].nb < nb || t[i].skinny != skinny) continue;
        if (t[i].dmax < 16 && t[i].dmax < need_diag) continue;
        if (exact_nb && (t[i].nb != exact_nb || t[i].kk != exact_kk)) continue;
        if (variant >= 0 && !t[i].fn[variant]) continue;
        if (variant < 0 && b32 && !t[i].fn[kB32Fly]) continue;
        if (variant < 0 && !b32 && !t[i].fn[kB64Fly]) continue;
        long cost = kept_pairs_before(t[i].na, t[i].nb, t[i].dmax, t[i].na, 0);     // MFMAs per 32x32x32 block
        // at equal MFMA count the deeper step wins (only instances made for int32 B have one)
        if (!best || cost < best_cost || (cost == best_cost && t[i].kk > best->kk)) { best = &t[i]; best_cost = cost; }
    }
    return best;
}

typedef std::tuple<const void *, long, long, int> OperandKey;     // (pointer, rows, K, element size)

// A range on its way from the device to the host behind the stream (calls that do not wait for their verdict).
struct PendingRange {
    hipEvent_t ev = nullptr;
    unsigned long long *host = nullptr;      // pinned: [minA, maxA, minB, maxB, verdict]
    OperandKey key_a, key_b;
    int nb_fixed = 0;                        // B came from prepared planes with this many digits (nothing of it was tracked)
    bool busy = false;
};

constexpr int kPendingSlots = 16;

struct RangeCache {
    std::mutex mu;
    std::map<OperandKey, int> limbs;         // operand -> digits its values needed when last seen
    std::map<OperandKey, int> partner_a;     // B operand -> digits of the A operand it was last multiplied with
    std::map<std::tuple<long, long, int>, int> by_shape;      // (rows, K, element size) -> digits of the last operand of that shape, wherever it lay
    unsigned long long *dev = nullptr;       // [minA, maxA, minB, maxB, verdict]
    unsigned char *planes = nullptr;         // digit planes of A, grown on demand, kept for the process lifetime
    size_t planes_bytes = 0;
    unsigned long long *mm = nullptr;        // per-workgroup ranges of the plane pre-pass
    size_t mm_count = 0;
    unsigned long long *wg = nullptr;        // per-workgroup ranges of the GEMM kernel
    size_t wg_count = 0;
    unsigned long long *partials = nullptr;  // partial sums of split tiles
    size_t partials_bytes = 0;
    int64_t *b_rows = nullptr;               // a small n-contiguous B rewritten with contiguous rows
    size_t b_rows_count = 0;
    int cus = 0;                             // compute units of the device
    PendingRange pending[kPendingSlots];
    unsigned long long *pinned = nullptr;
    int pending_head = 0;                    // next slot to use; slots are used and drained in ring order
    long guard_hits = 0;                     // calls whose speculation failed after they had returned
    int lookup(const OperandKey &k)
    {
        auto it = limbs.find(k);
        return it == limbs.end() ? 0 : it->second;
    }
    void store(const OperandKey &k, int n)
    {
        if (limbs.size() > 4096) limbs.clear();
        limbs[k] = n;
        if (by_shape.size() > 4096) by_shape.clear();
        by_shape[std::make_tuple(std::get<1>(k), std::get<2>(k), std::get<3>(k))] = n;
    }
    // An operand at an address never seen (or seen with another shape): what the last operand of its shape needed.  The
    // weights of one kind of projection need the same digits in every layer, and so do the activations that meet them.
    int lookup_shape(const OperandKey &k)
    {
        auto it = by_shape.find(std::make_tuple(std::get<1>(k), std::get<2>(k), std::get<3>(k)));
        return it == by_shape.end() ? 0 : it->second;
    }
    void store_pair(const OperandKey &ka, int na, const OperandKey &kb, int nb)
    {
        store(ka, na);
        store(kb, nb);
        if (partner_a.size() > 4096) partner_a.clear();
        partner_a[kb] = na;
    }
};

static RangeCache g_cache;

// Diagnosis switches, read from the environment once when the library is loaded (and again on zk_reload_env):
// ZK_GEMM_SYNC: every call waits for its own digit verdict; ZK_NO_TAIL_SPLIT: no split-K; ZK_VALU_FALLBACK: the guarded launch
// behind a speculative one is always the vector-ALU kernel; ZK_NO_STREAM32: grouped launches on int32 weights keep the general
// 32-row kernel; ZK_B_ROWS_MIN_MACS: product
// size from which a small n-contiguous int64 B is rewritten with contiguous rows first; ZK_SKINNY_MAX_M: rows up to
// which the 32-row tiles are used.
struct Switches { bool sync_verdict, no_tail_split, valu_fallback, no_stream32, no_pipe; double b_rows_min_macs; int skinny_max_m, planes_min_tiles_n, stream32_min_pairs; };
constexpr long kBRowsMinMacs = 1L << 32;
constexpr double kShapeGuessMaxMacs = 17179869184.0;        // 2^34: about 0.15 ms on the matrix pipe
// Rows up to which a product runs on the 32-row tiles (two of them from 33 rows on): measured against the 128-row tiles,
// 48 rows x [1536,7168] int32 34.1 against 38.1 us, 64 x [2048,7168] int64 37.6-39.4 against 41.2, 128 rows 56.8 against 45.1.
constexpr int kSkinnyMaxRows = 64;
static Switches read_switches()
{
    Switches s;
    s.sync_verdict = getenv("ZK_GEMM_SYNC") != nullptr;
    s.no_tail_split = getenv("ZK_NO_TAIL_SPLIT") != nullptr;
    s.valu_fallback = getenv("ZK_VALU_FALLBACK") != nullptr;
    s.no_stream32 = getenv("ZK_NO_STREAM32") != nullptr;
    s.no_pipe = getenv("ZK_NO_PIPE") != nullptr;
    const char *sp = getenv("ZK_STREAM32_MIN_PAIRS");
    s.stream32_min_pairs = sp ? atoi(sp) : 16;
    const char *m = getenv("ZK_B_ROWS_MIN_MACS");
    s.b_rows_min_macs = m ? atof(m) : (double)kBRowsMinMacs;
    const char *sk = getenv("ZK_SKINNY_MAX_M");
    s.skinny_max_m = sk ? atoi(sk) : kSkinnyMaxRows;
    const char *pt = getenv("ZK_PLANES_MIN_TILES_N");
    s.planes_min_tiles_n = pt ? atoi(pt) : 4;
    return s;
}
static Switches g_switches = read_switches();
void gemm_mfma_reload_switches() { g_switches = read_switches(); }

// Outcome of a launcher, derived from the call itself (never from the sticky error channel, which may still hold an
// error of an earlier, unrelated call): done, declined (nothing launched that the caller may not overwrite: it takes
// another route) or failed (an error was recorded).
enum Outcome { kDone = 0, kDeclined = 1, kFailed = -1 };

// Grows a device buffer kept until gemm_mfma_release_workspace.  kDeclined (buffer left empty) when memory is short.
template <typename T>
static Outcome grow(T *&buf, size_t &have, size_t need, const char *what)
{
    if (need <= have) return kDone;
    if (buf && hipFree(buf) != hipSuccess) { set_error(kLaunchFailure, "gemm: cannot release the %s", what); return kFailed; }
    buf = nullptr;
    have = 0;
    if (hipMalloc(&buf, need * sizeof(T)) != hipSuccess) { (void)hipGetLastError(); buf = nullptr; return kDeclined; }
    have = need;
    return kDone;
}

static bool read_range(unsigned long long *dev, int64_t (&out)[4])
{
    unsigned long long h[4];
    if (hipMemcpy(h, dev, sizeof(h), hipMemcpyDeviceToHost) != hipSuccess) return false;
    for (int i = 0; i < 4; i++) out[i] = (int64_t)(h[i] ^ kSignFlip);
    return true;
}

// Takes in the ranges that have arrived since the last call, oldest first.
static void drain_pending()
{
    for (int n = 0; n < kPendingSlots; n++) {
        PendingRange &s = g_cache.pending[(g_cache.pending_head + n) % kPendingSlots];
        if (!s.busy) continue;
        const hipError_t st = hipEventQuery(s.ev);
        if (st != hipSuccess) { (void)hipGetLastError(); if (st == hipErrorNotReady) continue; }
        if (st == hipSuccess) {
            const int64_t b_lo = (int64_t)(s.host[2] ^ kSignFlip), b_hi = (int64_t)(s.host[3] ^ kSignFlip);
            const int na_seen = limbs_needed((int64_t)(s.host[0] ^ kSignFlip), (int64_t)(s.host[1] ^ kSignFlip));
            if (b_lo <= b_hi) g_cache.store_pair(s.key_a, na_seen, s.key_b, limbs_needed(b_lo, b_hi));
            else if (s.nb_fixed) g_cache.store_pair(s.key_a, na_seen, s.key_b, s.nb_fixed);      // (a grouped launch on prepared planes)
            else g_cache.store(s.key_a, na_seen);            // B came from prepared planes: nothing of it was tracked
            if (s.host[4]) g_cache.guard_hits++;
        }
        s.busy = false;
    }
}

static int g_last_pairs = 0, g_last_prepared = 0;
static long g_streamed_calls = 0, g_pipe_calls = 0;
int gemm_mfma_last_pairs() { return g_last_pairs; }
int gemm_mfma_last_prepared() { return g_last_prepared; }
long gemm_mfma_grouped_streamed_calls() { return g_streamed_calls; }
long gemm_mfma_pipe_calls() { return g_pipe_calls; }

long gemm_mfma_guard_hits()
{
    std::lock_guard<std::mutex> lock(g_cache.mu);
    drain_pending();
    return g_cache.guard_hits;
}

static bool init_cache()
{
    if (g_cache.dev) return true;
    // [minA, maxA, minB, maxB, verdict, fold ticket, -, -] and the partial results of the folding workgroups
    const size_t dev_bytes = (8 + 4 * kFoldParts) * sizeof(unsigned long long);
    if (hipMalloc(&g_cache.dev, dev_bytes) != hipSuccess || hipMemset(g_cache.dev, 0, dev_bytes) != hipSuccess) {
        g_cache.dev = nullptr;
        set_error(kLaunchFailure, "gemm: cannot allocate the range buffer");
        return false;
    }
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    g_cache.cus = n;
    // without the pinned slots every call simply waits for its own verdict
    if (hipHostMalloc(&g_cache.pinned, kPendingSlots * 8 * sizeof(unsigned long long), hipHostMallocDefault) == hipSuccess) {
        for (int i = 0; i < kPendingSlots; i++) {
            g_cache.pending[i].host = g_cache.pinned + 8 * i;
            if (hipEventCreateWithFlags(&g_cache.pending[i].ev, hipEventDisableTiming) != hipSuccess) g_cache.pending[i].ev = nullptr;
        }
    } else {
        (void)hipGetLastError();
        g_cache.pinned = nullptr;
    }
    return true;
}

static FoldArgs make_fold(const unsigned long long *mm, long mm_count, const unsigned long long *wg, long wg_count,
                          unsigned long long *range, int na, int nb, unsigned long long *host_copy)
{
    long parts = (mm_count + wg_count + kFoldSlotsPerPart - 1) / kFoldSlotsPerPart;
    parts = parts < 1 ? 1 : (parts > kFoldParts ? kFoldParts : parts);
    return FoldArgs{ mm, mm_count, wg, wg_count, range, na, nb, host_copy, (int)parts, g_cache.dev + 8 };
}

// ---- weights prepared once ------------------------------------------------------------------------------
// Model weights do not change between calls.  `gemm_mfma_prepare` splits an int64 weight matrix (or every matrix of a
// device table of pointers, the experts of a layer) into digit planes in MFMA fragment order once, with the digit
// count its exact range needs; later launches whose B is that pointer copy the planes into LDS instead of splitting B
// in every tile (and read NB bytes per weight instead of 8).  The original matrix stays the caller's and is what the
// guarded vector-ALU fallback reads; the caller must not change it while it is prepared.
struct PreparedB {
    unsigned char *planes = nullptr;     // per matrix: [nsub][ksteps][nb] blocks of 1 KB
    const void **table = nullptr;        // device array: the planes of every group (tables only)
    int groups = 0, N = 0, K = 0, nb = 0, nsub = 0, ksteps = 0, b32 = 0;
    int kk = 1;                          // MFMA depths per step of the kernels the planes were ordered for
};
static std::map<const void *, PreparedB> g_prepared;

template <typename T>
static __global__ __launch_bounds__(256) void range_exact_kernel(const T *__restrict__ x, long n, unsigned long long *out)
{
    MinMax r = { INT64_MAX, INT64_MIN };
    // 16-byte pieces, four in flight per thread, then whatever is left (n and the pointer need not be aligned)
    constexpr int PER = 16 / sizeof(T);
    const long head = ((uintptr_t)x & 15) ? n : 0;                       // unaligned: everything goes element by element
    const long pieces = (n - head) / PER;
    const v4i *xv = reinterpret_cast<const v4i *>(x);
    for (long q0 = (long)blockIdx.x * 1024 + threadIdx.x; q0 < pieces; q0 += (long)gridDim.x * 1024) {
        v4i t[4];
#pragma unroll
        for (int u = 0; u < 4; u++) t[u] = q0 + 256 * u < pieces ? __builtin_nontemporal_load(xv + q0 + 256 * u) : xv[0];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (sizeof(T) == 8) {
                mm_update(r, (int64_t)(((uint64_t)(uint32_t)t[u][1] << 32) | (uint32_t)t[u][0]));
                mm_update(r, (int64_t)(((uint64_t)(uint32_t)t[u][3] << 32) | (uint32_t)t[u][2]));
            } else {
#pragma unroll
                for (int z = 0; z < 4; z++) mm_update(r, (int64_t)t[u][z]);
            }
        }
    }
    for (long i = (head ? 0 : pieces * PER) + (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) mm_update(r, (int64_t)x[i]);
    r = mm_wave(r);
    if ((threadIdx.x & 63) == 0 && r.lo <= r.hi) {
        atomicMin(out, (unsigned long long)r.lo ^ kSignFlip);
        atomicMax(out + 1, (unsigned long long)r.hi ^ kSignFlip);
    }
}

static void release_prepared(PreparedB &pb)
{
    if (pb.planes) (void)hipFree(pb.planes);
    if (pb.table) (void)hipFree((void *)pb.table);
    pb = PreparedB();
}

bool gemm_mfma_is_prepared(const void *B)
{
    std::lock_guard<std::mutex> lock(g_cache.mu);
    return g_prepared.count(B) != 0;
}

void gemm_mfma_release(const void *B)
{
    std::lock_guard<std::mutex> lock(g_cache.mu);
    auto it = g_prepared.find(B);
    if (it == g_prepared.end()) return;
    (void)hipDeviceSynchronize();              // launches that read the planes may still be under way
    release_prepared(it->second);
    g_prepared.erase(it);
}

int gemm_mfma_prepare(const void *B, int b32, int groups, int N, int K)
{
    const char *name = "zk_gemm_prepare_weights";
    if (!B || groups < 0 || groups > 65535 || N < 1 || K < 1) { set_error(kBadArgument, "%s: bad argument", name); return 1; }
    std::lock_guard<std::mutex> lock(g_cache.mu);
    if (!init_cache()) return 1;
    {
        auto it = g_prepared.find(B);
        if (it != g_prepared.end()) { (void)hipDeviceSynchronize(); release_prepared(it->second); g_prepared.erase(it); }
    }
    const int count = groups > 0 ? groups : 1;
    std::vector<const void *> mats((size_t)count, B);
    if (groups > 0 && hipMemcpy(mats.data(), B, (size_t)count * sizeof(void *), hipMemcpyDeviceToHost) != hipSuccess) {
        set_error(kLaunchFailure, "%s: cannot read the pointer table", name);
        return 1;
    }
    for (int i = 0; i < count; i++)
        if (!mats[i]) { set_error(kBadArgument, "%s: null matrix in the table", name); return 1; }
    // the exact range of all the matrices fixes one digit count for them
    const long elems = (long)N * K;
    range_reset_kernel<<<1, 64, 0, 0>>>(g_cache.dev);
    const unsigned rgrid = (unsigned)(elems / 256 + 1 < 2048 ? elems / 256 + 1 : 2048);
    for (int i = 0; i < count; i++) {
        if (b32) range_exact_kernel<int32_t><<<rgrid, 256, 0, 0>>>(reinterpret_cast<const int32_t *>(mats[i]), elems, g_cache.dev);
        else range_exact_kernel<int64_t><<<rgrid, 256, 0, 0>>>(reinterpret_cast<const int64_t *>(mats[i]), elems, g_cache.dev);
    }
    int64_t r[4];
    if (!read_range(g_cache.dev, r)) { set_error(kLaunchFailure, "%s: range readback failed", name); return 1; }
    const int need = limbs_needed(r[0], r[1]);
    PreparedB pb;
    pb.groups = groups; pb.N = N; pb.K = K; pb.b32 = b32 ? 1 : 0;
    pb.nb = need <= 3 ? 3 : (need <= 5 ? need : 9);              // digit counts the kernels are built for
    // the experts' three- and four-digit planes go to kernels with two depths per step (the k-order inside a step follows it)
    pb.kk = (groups > 0 && pb.nb <= 4) ? 2 : 1;
    pb.nsub = (N + 31) / 32;
    pb.ksteps = ((K + 32 * pb.kk - 1) / (32 * pb.kk)) * pb.kk;
    const size_t per = (size_t)pb.nsub * pb.ksteps * pb.nb * 1024;
    if (hipMalloc(&pb.planes, per * count) != hipSuccess) {
        (void)hipGetLastError();
        set_error(kLaunchFailure, "%s: cannot allocate %zu bytes of digit planes", name, per * count);
        return 1;
    }
    if (groups > 0) {
        std::vector<const void *> bases((size_t)count);
        for (int i = 0; i < count; i++) bases[i] = pb.planes + per * i;
        if (hipMalloc((void **)&pb.table, (size_t)count * sizeof(void *)) != hipSuccess ||
            hipMemcpy((void *)pb.table, bases.data(), (size_t)count * sizeof(void *), hipMemcpyHostToDevice) != hipSuccess) {
            (void)hipGetLastError();
            release_prepared(pb);
            set_error(kLaunchFailure, "%s: cannot allocate the table of planes", name);
            return 1;
        }
    }
    // the pre-pass that splits A in fragment order does the same for the rows of a weight matrix (64 rows per workgroup)
    const int rows_per_wg = 256 / (4 * pb.kk);
    const dim3 grid((unsigned)(pb.ksteps / pb.kk), (unsigned)((pb.nsub * 32 + rows_per_wg - 1) / rows_per_wg), 1);
    if (grow(g_cache.mm, g_cache.mm_count, (size_t)grid.x * grid.y * 2, "range scratch") != kDone) {
        release_prepared(pb);
        set_error(kLaunchFailure, "%s: cannot allocate the range scratch", name);
        return 1;
    }
    MfmaParams q = {};
    q.lda = K; q.sA = 0; q.M = N; q.K = K;
    for (int i = 0; i < count; i++) {
        q.A = reinterpret_cast<const int64_t *>(mats[i]);
        unsigned char *dst = pb.planes + per * i;
#define ZK_PLANES(NB_) do { if (b32) a_planes_kernel<NB_, 2, 1, true><<<grid, dim3(256), 0, 0>>>(q, dst, pb.nsub, pb.ksteps, g_cache.mm); \
                           else a_planes_kernel<NB_, 2, 1, false><<<grid, dim3(256), 0, 0>>>(q, dst, pb.nsub, pb.ksteps, g_cache.mm); } while (0)
        switch (pb.nb) {
#define ZK_PLANES2(NB_) do { if (b32) a_planes_kernel<NB_, 2, 2, true><<<grid, dim3(256), 0, 0>>>(q, dst, pb.nsub, pb.ksteps, g_cache.mm); \
                            else a_planes_kernel<NB_, 2, 2, false><<<grid, dim3(256), 0, 0>>>(q, dst, pb.nsub, pb.ksteps, g_cache.mm); } while (0)
        case 3: if (pb.kk == 2) ZK_PLANES2(3); else ZK_PLANES(3); break;
        case 4: if (pb.kk == 2) ZK_PLANES2(4); else ZK_PLANES(4); break;
#undef ZK_PLANES2
        case 5: ZK_PLANES(5); break;
        default: ZK_PLANES(9); break;
        }
#undef ZK_PLANES
    }
    if (hipGetLastError() != hipSuccess || hipDeviceSynchronize() != hipSuccess) {
        release_prepared(pb);
        set_error(kLaunchFailure, "%s: the plane pre-pass failed", name);
        return 1;
    }
    g_prepared[B] = pb;
    return 0;
}

// Device memory the GEMM path holds right now: its scratch buffers, and the digit planes of prepared weights.
size_t gemm_mfma_workspace_bytes(size_t *prepared_bytes)
{
    std::lock_guard<std::mutex> lock(g_cache.mu);
    size_t scratch = g_cache.dev ? (8 + 4 * kFoldParts) * sizeof(unsigned long long) : 0;
    scratch += g_cache.planes_bytes + (g_cache.mm_count + g_cache.wg_count + g_cache.partials_bytes) * sizeof(unsigned long long) +
               g_cache.b_rows_count * sizeof(int64_t);
    size_t prepared = 0;
    for (const auto &kv : g_prepared) {
        const PreparedB &pb = kv.second;
        const size_t count = pb.groups > 0 ? (size_t)pb.groups : 1;
        prepared += (size_t)pb.nsub * pb.ksteps * pb.nb * 1024 * count + (pb.table ? count * sizeof(void *) : 0);
    }
    if (prepared_bytes) *prepared_bytes = prepared;
    return scratch;
}

// Gives the scratch buffers back (they grow again on demand).  Waits for the device first: launches that use them may
// still be under way.  Prepared weights stay (zk_gemm_release_weights returns those).
void gemm_mfma_release_workspace()
{
    std::lock_guard<std::mutex> lock(g_cache.mu);
    (void)hipDeviceSynchronize();
    drain_pending();
    if (g_cache.planes) (void)hipFree(g_cache.planes);
    if (g_cache.mm) (void)hipFree(g_cache.mm);
    if (g_cache.wg) (void)hipFree(g_cache.wg);
    if (g_cache.partials) (void)hipFree(g_cache.partials);
    if (g_cache.b_rows) (void)hipFree(g_cache.b_rows);
    g_cache.planes = nullptr; g_cache.planes_bytes = 0;
    g_cache.mm = nullptr; g_cache.mm_count = 0;
    g_cache.wg = nullptr; g_cache.wg_count = 0;
    g_cache.partials = nullptr; g_cache.partials_bytes = 0;
    g_cache.b_rows = nullptr; g_cache.b_rows_count = 0;
}

// B[g][k][n] (n contiguous) -> out[g][n][k]: 32x32 tiles through LDS, both sides coalesced
__global__ __launch_bounds__(256) void b_rows_kernel(const int64_t *__restrict__ B, long ldbk, long sB, int64_t *__restrict__ out, int N, int K)
{
    __shared__ int64_t tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int n0 = blockIdx.x * 32, k0 = blockIdx.y * 32;
    const int64_t *src = B + (long)blockIdx.z * sB;
    int64_t *dst = out + (long)blockIdx.z * N * K;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int k = k0 + ty + 8 * i, n = n0 + tx;
        tile[ty + 8 * i][tx] = (k < K && n < N) ? src[(long)k * ldbk + n] : 0;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int n = n0 + ty + 8 * i, k = k0 + tx;
        if (n < N && k < K) dst[(long)n * K + k] = tile[tx][ty + 8 * i];
    }
}

// An n-contiguous int64 B that is small next to the product (the values of an attention step against all the
// probabilities, `bsht,btc->bshc`) is worth rewriting with contiguous rows first: the row-major kernels read it with
// 16-byte loads and take A from digit planes (measured at S = T = 1024, 128 heads: 1.67 -> 1.45 ms, the rewrite 9 us).
constexpr long kBRowsMaxElements = 8L << 20;         // 64 MB

// The launch behind a speculative one: it does nothing unless the verdict word says that the digit counts did not cover
// the operands, and then computes every output again.  Row-major B without a divisor: the widest MFMA instance (nine
// digits hold every int64, five every int32; config 4 with stale three-digit guesses: 4 ms where the vector-ALU tiles
// take 35), one workgroup per compute unit walking the tiles.  Everything else, and a K beyond what its int32
// accumulators take in one piece: the vector-ALU tiles.
static Outcome launch_guarded_fallback(const GemmDesc &d, const MfmaParams &spec, int b_shift)
{
    // (an n-contiguous B that the speculative launch read through its row-major copy is read through that copy here too)
    const bool b_copied = spec.B == (const void *)g_cache.b_rows && g_cache.b_rows != nullptr;
    const bool row_major = b_copied || !(d.ldbn == 1 && d.ldbk != 1);
    const Instance *wide = (row_major && b_shift == 0 && !g_switches.valu_fallback) ? pick_instance(9, d.b32 ? 5 : 9, d.b32 != 0, false, 16) : nullptr;
    MfmaKernel fn = wide ? wide->guarded[d.b32 ? 1 : 0] : nullptr;
    if (fn) {
        const long pairs = wide->na < wide->nb ? wide->na : wide->nb;
        const int ksteps = ((d.K + 32 * wide->kk - 1) / (32 * wide->kk)) * wide->kk;
        if (pairs * ksteps * 32 * 16384 > 0x7FFFFFFFL) fn = nullptr;
    }
    MfmaParams q = spec;
    if (fn) {
        // the caller's operands, not digit planes
        q.A = d.A; q.lda = d.lda; q.sA = d.sA;
        if (!b_copied) { q.B = d.B; q.ldbn = d.ldbn; q.ldbk = d.ldbk; q.sB = d.sB; }
        q.a_planes = nullptr; q.a_msub = 0; q.a_ksteps = 0; q.b_nsub = 0; q.b_ksteps = 0;
        q.tiles_m = (d.M + wide->bm - 1) / wide->bm;
        q.tiles_n = (d.N + wide->bn - 1) / wide->bn;
        const long total = (long)q.tiles_m * q.tiles_n * d.G;
        if (total > 0x7FFFFFFFL / 8) fn = nullptr;
        else {
            q.main_tiles = (int)total; q.split = 1; q.tail_xcd = 0; q.partials = nullptr; q.part64 = 0; q.n_fastest = 0;
            q.guard = spec.range + 4;
            q.walk_blocks = (int)total;
            // (the range slots of the speculative launch have been folded by now: the fallback's tracking may overwrite them)
            const Outcome got = grow(g_cache.wg, g_cache.wg_count, (size_t)total * 4, "range slots");
            if (got == kFailed) return kFailed;
            if (got == kDeclined) fn = nullptr;
            q.wg_range = g_cache.wg;
        }
    }
    if (!fn) {
        gemm_valu_launch(d, spec.range + 4);
        return kDone;
    }
    const size_t lds = 2 * (size_t)wide->kk * ((wide->bm / 32) * wide->na + (wide->bn / 32) * wide->nb) * 1024 + 9 * 1024 + 16;
    static std::set<const void *> lds_raised;
    if (lds > 64 * 1024 && !lds_raised.count((const void *)fn)) {
        if (hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
            set_error(kLaunchFailure, "gemm: cannot raise the LDS limit to %zu bytes", lds);
            return kFailed;
        }
        lds_raised.insert((const void *)fn);
    }
    const long grid = q.walk_blocks < g_cache.cus ? q.walk_blocks : g_cache.cus;
    fn<<<dim3((unsigned)grid), dim3((unsigned)wide->threads), lds, 0>>>(q);
    if (hipGetLastError() != hipSuccess) { set_error(kLaunchFailure, "gemm: guarded MFMA launch failed"); return kFailed; }
    return kDone;
}

int gemm_mfma_launch(const GemmDesc &d, int *limbs_a, int *limbs_b)
{
    // Operand divisors: a power of two on B is folded into the digit split of the 32-row kernels (the head projection
    // divides its weights by 256, inference/model.py:1519, and runs on the last token only); anything else: VALU path.
    int b_shift = 0;
    if (d.a_rs != 1) return kDeclined;
    if (d.b_rs != 1) {
        if (d.b_rs <= 0 || (d.b_rs & (d.b_rs - 1)) != 0 || d.M > 32) return kDeclined;
        while (((int64_t)1 << b_shift) < d.b_rs) b_shift++;
    }
    if (d.K <= 0 || d.M <= 0 || d.N <= 0 || d.G <= 0) return kDeclined;
    if (d.G > 65535) return kDeclined;
    bool kmajor = d.ldbn == 1 && d.ldbk != 1;
    std::lock_guard<std::mutex> lock(g_cache.mu);
    if (!init_cache()) return kFailed;
    drain_pending();

    MfmaParams p = {};
    p.A = d.A; p.B = d.B; p.C = d.C; p.R = d.R;
    p.lda = d.lda; p.sA = d.sA; p.ldbn = d.ldbn; p.ldbk = d.ldbk; p.sB = d.sB; p.ldc = d.ldc; p.sC = d.sC;
    // B prepared beforehand: its planes stand in for it, its digit count is exact
    const PreparedB *prep = nullptr;
    {
        auto it = g_prepared.find(d.B);
        if (it != g_prepared.end() && it->second.groups == 0 && it->second.b32 == (d.b32 ? 1 : 0) && !kmajor && b_shift == 0 && d.sB == 0 &&
            d.ldbk == 1 && d.ldbn == d.K && it->second.N == d.N && it->second.K == d.K)
            prep = &it->second;
    }
    const long b_batches = d.sB != 0 ? d.G : 1;
    if (kmajor && !d.b32 && d.M > 32 && b_batches * d.N * d.K <= kBRowsMaxElements &&
        (double)d.G * d.M * d.N * d.K >= g_switches.b_rows_min_macs) {
        // (without memory for the copy the n-contiguous kernels run as before)
        const Outcome got = grow(g_cache.b_rows, g_cache.b_rows_count, (size_t)(b_batches * d.N * d.K), "row-major copy of B");
        if (got == kDone) {
            const dim3 grid((unsigned)((d.N + 31) / 32), (unsigned)((d.K + 31) / 32), (unsigned)b_batches);
            b_rows_kernel<<<grid, dim3(256), 0, 0>>>(reinterpret_cast<const int64_t *>(d.B), d.ldbk, d.sB, g_cache.b_rows, d.N, d.K);
            p.B = g_cache.b_rows; p.ldbn = d.K; p.ldbk = 1; p.sB = d.sB != 0 ? (long)d.N * d.K : 0;
            kmajor = false;
        } else if (got == kFailed) {
            return kFailed;
        }
    }
    p.M = d.M; p.N = d.N; p.K = d.K; p.shift = d.shift; p.init = d.init;
    p.range = g_cache.dev;
    p.verify_b_all_batches = d.sB != 0;
    p.b_shift = b_shift;

    // (a divided B has another range than the raw one: the shift is part of its key)
    const OperandKey key_a(d.A, (long)d.G * d.M, d.K, 8), key_b(d.B, d.N, d.K, (d.b32 ? 4 : 8) | (b_shift << 8));
    int na = g_cache.lookup(key_a), nb = prep ? prep->nb : g_cache.lookup(key_b);
    // Activations gathered into a fresh buffer for a known weight matrix (the experts of a MoE layer): guess the
    // digits the last activations multiplied with that matrix needed.  A wrong guess costs one guarded recomputation.
    if (!na && nb) {
        auto it = g_cache.partner_a.find(key_b);
        if (it != g_cache.partner_a.end()) na = it->second;
    }
    // Operands at addresses never seen: for products below kShapeGuessMaxMacs the digits of the last operands of the
    // same shapes stand in (a wrong guess costs such a product less than the wait for a sample would: the reference's
    // driver builds every layer anew, generate.py:227-238, so most of its calls come with new or recycled addresses);
    // larger products, and shapes never seen, are sampled, which waits for the stream once.
    if ((!na || !nb) && (double)d.G * d.M * d.N * d.K < kShapeGuessMaxMacs) {
        if (!na) na = g_cache.lookup_shape(key_a);
        if (!nb) nb = g_cache.lookup_shape(key_b);
    }
    // No call waits for its verdict (unless no slot is free for the range to travel in, or ZK_GEMM_SYNC asks for it): a
    // guarded launch behind the product redoes it with digits that cover everything if the verdict is bad.
    PendingRange *slot = nullptr;
    if (g_cache.pinned && !g_switches.sync_verdict) {
        PendingRange &s = g_cache.pending[g_cache.pending_head];
        if (!s.busy && s.ev) slot = &s;
    }
    if (!na || !nb) {
        p.tiles_m = p.tiles_n = 1;
        range_reset_kernel<<<1, 64, 0, 0>>>(p.range);
        range_sample_kernel<<<1, 256, 0, 0>>>(p, d.b32, d.G, 0);
        range_sample_kernel<<<1, 256, 0, 0>>>(p, d.b32, d.G, 1);
        int64_t r[4];
        if (!read_range(p.range, r)) { set_error(kLaunchFailure, "gemm: range readback failed"); return kFailed; }
        if (!na) na = limbs_needed(r[0], r[1]);
        if (!nb) nb = limbs_needed(r[2], r[3]);
    }
    if (prep) { p.B = prep->planes; p.b_nsub = prep->nsub; p.b_ksteps = prep->ksteps; }

    for (int attempt = 0; attempt < 3; attempt++) {
        // the stored bits are [shift, shift + 64) of the sum (the remainder lies below them)
        const int need_diag = (d.shift + 64 + 7) / 8;
        // (the kernels that read planes never see B's element type: they are the int64 forms)
        const Instance *inst = d.M <= g_switches.skinny_max_m ? pick_instance(na, nb, d.b32 != 0 && !prep, true, need_diag, prep ? prep->nb : 0, prep ? kB64FlyBPlanes : -1) : nullptr;
        if (!inst) inst = pick_instance(na, nb, d.b32 != 0 && !prep, false, need_diag, prep ? prep->nb : 0, prep ? kB64PlanesBoth : -1);
        if (!inst && prep) {
            // no kernel with exactly the planes' digit count covers A: this call splits the original B like any other
            // (nb, the planes' count, covers B)
            prep = nullptr;
            p.B = d.B;
            inst = d.M <= g_switches.skinny_max_m ? pick_instance(na, nb, d.b32 != 0, true, need_diag) : nullptr;
            if (!inst) inst = pick_instance(na, nb, d.b32 != 0, false, need_diag);
        }
        if (!inst) return kDeclined;
        // int32 accumulators: at most min(NA,NB) digit pairs per diagonal, each product at most 2^14 in magnitude
        const long pairs = inst->na < inst->nb ? inst->na : inst->nb;
        const int ksteps = ((d.K + 32 * inst->kk - 1) / (32 * inst->kk)) * inst->kk;     // 32-k steps, padded
        // (a K beyond that bound is cut into slices that respect it: every tile is then split, see below)
        const bool k_over = pairs * ksteps * 32 * 16384 > 0x7FFFFFFFL;
        const int BM = inst->bm, BN = inst->bn;
        p.tiles_m = (d.M + BM - 1) / BM;
        p.tiles_n = (d.N + BN - 1) / BN;
        // A B operand that stays in L2 whatever the order (the MLA einsums: a KV cache or one head's weights against
        // a hundred thousand rows) lets the tile columns move fastest, so that each A tile is streamed once
        const size_t b_bytes = (size_t)d.N * d.K * (d.b32 ? 4 : 8);
        p.n_fastest = (b_bytes <= ((size_t)8 << 20) && p.tiles_n > 1 && p.tiles_m > 1) ? 1 : 0;
        const long per_batch = (long)p.tiles_m * p.tiles_n;
        if (per_batch > 0x7FFFFFFFL) return kDeclined;
        const long total = per_batch * d.G;
        if (total > 0x7FFFFFFFL / 8) return kDeclined;
        // A is pre-split into digit planes when enough column tiles reuse it to pay for the extra pass (never for the
        // 32-row tiles: splitting a handful of rows on the fly is cheaper than another kernel in front)
        // (nor for a launch with fewer tiles than compute units: its tiles are cut along K, every workgroup splits a short
        // slice of A, and the pre-pass would be a launch of its own in front: 128 rows x [2048,7168] 43.8 -> 42.4 us)
        const bool use_planes = !kmajor && ((p.tiles_n >= g_switches.planes_min_tiles_n && total >= g_cache.cus) || prep) && !inst->skinny;
        if (b_shift && (kmajor || !inst->skinny)) return kDeclined;
        const int variant = prep ? (inst->skinny ? kB64FlyBPlanes : kB64PlanesBoth)
                          : b_shift ? (d.b32 ? kB32FlyRs : kB64FlyRs)
                          : kmajor ? (d.b32 ? kB32KmajorFly : kB64KmajorFly)
                                   : (d.b32 ? (use_planes ? kB32Planes : kB32Fly) : (use_planes ? kB64Planes : kB64Fly));
        MfmaKernel fn = inst->fn[variant];
        if (!fn) return kDeclined;
        // planes on both sides and the 128 x 128 tile: the software-pipelined form (gemm_mfma_pipe.h; same tiles, planes,
        // partial sums and outputs)
        size_t pipe_lds = 0;
        if (variant == kB64PlanesBoth && !g_switches.no_pipe && BM == 128 && BN == 128 && inst->kk == 1) {
            if (MfmaKernel pfn = pipe_kernel(inst->na, inst->nb)) { fn = pfn; pipe_lds = pipe_lds_size(inst->na, inst->nb); }
        }

        // Split-K: a launch smaller than the device is cut into `split` slices of K per tile, each a workgroup of
        // its own; with more tiles than compute units the same is done for the tiles of the last, partial round
        // only.  The slices leave raw partial sums and a small kernel adds them.
        const int steps = (d.K + 32 * inst->kk - 1) / (32 * inst->kk);
        int tail = (int)(total % g_cache.cus), split = 1;
        p.main_tiles = (int)total;
        p.split = 1;
        p.tail_xcd = 0;
        p.partials = nullptr;
        p.part64 = 0;
        p.finish_rq = 4;
        if (!g_switches.no_tail_split) {
            if (total < g_cache.cus) {
                tail = (int)total;
                split = g_cache.cus / tail;
                if (split > 64) split = 64;
                if (split > steps / 4) split = steps / 4;
                p.finish_rq = 16;
            } else if (inst->skinny && total < 8L * g_cache.cus) {
                // a few rows against many columns is a weight stream: more, shorter workgroups keep more of it in
                // flight and even out the last round (the partial sums of so few rows cost next to nothing)
                tail = (int)total;
                split = (int)((8L * g_cache.cus + total - 1) / total);
                if (split > 64) split = 64;
                if (split > steps / 4) split = steps / 4;
                p.finish_rq = 16;
            } else if (tail > 0 && tail <= g_cache.cus / 2) {
                split = g_cache.cus / tail;
                if (split > 8) split = 8;
                if (split > steps / 8) split = steps / 8;
            }
        }
        if (k_over) {
            // every tile in slices short enough for the int32 accumulators; without room for the partial sums (or with
            // the split switched off) the vector-ALU path takes the product
            int min_split = 2;
            while (pairs * ((steps + min_split - 1) / min_split) * 32 * inst->kk * 16384 > 0x7FFFFFFFL) min_split++;
            if (g_switches.no_tail_split || min_split > steps) return kDeclined;
            if (tail != (int)total || split < min_split) {
                tail = (int)total;
                split = min_split;
                p.finish_rq = 4;
            }
            if ((size_t)tail * split * BM * BN * 16 > ((size_t)2 << 30)) return kDeclined;
        }
        if (split >= 2) {
            // |sum| < K * 2^(8(NA+NB)-2): below 2^62 the low word alone carries a partial sum
            int kbits = 0;
            while ((1L << kbits) < (long)ksteps * 32) kbits++;
            const bool part64 = 8 * (inst->na + inst->nb) - 2 + kbits <= 62;
            const size_t need = (size_t)tail * split * BM * BN * (part64 ? 1 : 2);
            const Outcome got = grow(g_cache.partials, g_cache.partials_bytes, need, "partial-sum buffer");
            if (got == kDone) {
                p.main_tiles = (int)(total - tail);
                p.split = split;
                p.tail_xcd = (!p.n_fastest && d.G == 1 && tail % p.tiles_m == 0 && p.main_tiles % 8 == 0 &&
                              ((long)tail * split) % (8L * p.tiles_m) == 0) ? 1 : 0;
                p.partials = g_cache.partials;
                p.part64 = part64 ? 1 : 0;
            } else if (got == kFailed) return kFailed;
            else if (k_over) return kDeclined;
        }
        const long blocks = (long)p.main_tiles + (total - p.main_tiles) * p.split;
        // (room for the guarded fallback's 64 x 64 tiles as well, so that it never has to regrow the buffer)
        const long fb_blocks = (long)((d.M + 63) / 64) * ((d.N + 63) / 64) * d.G;
        if (const Outcome got = grow(g_cache.wg, g_cache.wg_count, (size_t)(blocks > fb_blocks ? blocks : fb_blocks) * 4, "range slots")) return got;
        p.wg_range = g_cache.wg;

        long plane_wgs = 0;
        p.a_planes = nullptr; p.a_msub = 0; p.a_ksteps = 0;
        if (use_planes) {
            const int msub = p.tiles_m * (BM / 32);
            const size_t need = (size_t)d.G * msub * ksteps * inst->na * 1024;
            // not enough memory for planes: the caller uses the VALU path
            if (const Outcome got = grow(g_cache.planes, g_cache.planes_bytes, need, "digit-plane buffer")) return got;
            p.a_planes = g_cache.planes; p.a_msub = msub; p.a_ksteps = ksteps;
            const int rows_per_wg = 256 / (4 * inst->kk);
            const dim3 pgrid((unsigned)(ksteps / inst->kk), (unsigned)((msub * 32 + rows_per_wg - 1) / rows_per_wg), (unsigned)d.G);
            plane_wgs = (long)pgrid.x * pgrid.y * pgrid.z;
            if (const Outcome got = grow(g_cache.mm, g_cache.mm_count, (size_t)plane_wgs * 2, "range scratch")) return got;
            // (the owned-k pattern of the planes of A follows the kernel that reads them: prepared planes of B go with the int64 forms)
            inst->planes[(d.b32 && !prep) ? 1 : 0]<<<pgrid, dim3(256), 0, 0>>>(p, g_cache.planes, msub, ksteps, g_cache.mm);
        }
        const size_t lds = pipe_lds ? pipe_lds : 2 * (size_t)inst->kk * ((BM / 32) * inst->na + (BN / 32) * inst->nb) * 1024 + 9 * 1024 + 16;
        static std::set<const void *> lds_raised;
        if (lds > 64 * 1024 && !lds_raised.count((const void *)fn)) {
            if (hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
                set_error(kLaunchFailure, "gemm: cannot raise the LDS limit to %zu bytes", lds);
                return kFailed;
            }
            lds_raised.insert((const void *)fn);
        }
        fn<<<dim3((unsigned)blocks), dim3((unsigned)inst->threads), lds, 0>>>(p);
        g_last_pairs = kept_pairs_before(inst->na, inst->nb, inst->dmax, inst->na, 0);
        g_last_prepared = prep ? 1 : 0;
        if (pipe_lds) g_pipe_calls++;
        {
            const hipError_t err = hipGetLastError();
            if (err != hipSuccess) {
                set_error(kLaunchFailure, "gemm: MFMA kernel launch failed (%s; digits %d,%d, %ld workgroups of %d threads, %zu bytes of LDS)",
                          hipGetErrorString(err), inst->na, inst->nb, blocks, inst->threads, lds);
                return kFailed;
            }
        }
        const FoldArgs fold = make_fold(g_cache.mm, plane_wgs, g_cache.wg, blocks, p.range, inst->na, inst->nb, slot ? slot->host : nullptr);
        if (p.split > 1) {
            inst->finish<<<dim3((unsigned)((total - p.main_tiles) * p.finish_rq + fold.parts)), dim3((unsigned)inst->threads), 0, 0>>>(p, fold);
            if (hipGetLastError() != hipSuccess) { set_error(kLaunchFailure, "gemm: split finish launch failed"); return kFailed; }
        } else {
            range_fold_kernel<<<dim3((unsigned)fold.parts), 256, 0, 0>>>(fold);
        }
        *limbs_a = inst->na;
        *limbs_b = inst->nb;
        if (slot) {
            // no waiting: a guarded launch redoes the product if the verdict is bad, the range follows later
            if (const Outcome got = launch_guarded_fallback(d, p, b_shift)) return got;
            if (hipEventRecord(slot->ev, 0) == hipSuccess) {
                slot->key_a = key_a;
                slot->key_b = key_b;
                slot->nb_fixed = prep ? prep->nb : 0;       // (the slots are shared with the grouped launches, which set it too)
                slot->busy = true;
                g_cache.pending_head = (g_cache.pending_head + 1) % kPendingSlots;
            } else {
                (void)hipGetLastError();
            }
            return kDone;
        }
        int64_t r[4];
        if (!read_range(p.range, r)) { set_error(kLaunchFailure, "gemm: range readback failed"); return kFailed; }
        const int need_a = limbs_needed(r[0], r[1]), need_b = prep ? prep->nb : limbs_needed(r[2], r[3]);
        g_cache.store_pair(key_a, need_a, key_b, need_b);
        if (need_a <= inst->na && need_b <= inst->nb) return kDone;
        na = need_a;
        nb = need_b;
    }
    set_error(kLaunchFailure, "gemm: digit count did not settle");
    return kFailed;
}

int gemm_mfma_grouped(const GroupedDesc &d, int *limbs_a, int *limbs_b)
{
    if (d.K <= 0 || d.N <= 0 || d.rows <= 0 || d.groups <= 0) return 1;
    std::lock_guard<std::mutex> lock(g_cache.mu);
    if (!init_cache()) return -1;
    drain_pending();

    MfmaParams p = {};
    p.A = d.A; p.B = nullptr; p.C = d.C; p.R = d.R;
    p.lda = d.lda; p.sA = 0; p.ldbn = d.K; p.ldbk = 1; p.sB = 0; p.ldc = d.ldc; p.sC = 0;
    p.M = d.rows; p.N = d.N; p.K = d.K; p.shift = d.shift; p.init = d.init;
    p.range = g_cache.dev;
    p.tiles_m = 1;
    p.split = 1; p.finish_rq = 4;
    p.grp_seg = d.seg; p.grp_tiles = d.tiles; p.grp_ntiles = d.ntiles; p.grp_b = d.B;

    // digits: what these operands needed last time, else the widest the 32-row kernels have
    const OperandKey key_a(d.A, (long)d.rows, d.K, 8), key_b(d.B, (long)d.groups * d.N, d.K, d.b32 ? 4 : 8);
    // the experts' weights prepared beforehand (the table pointer is the key): planes instead of B, an exact digit count
    const PreparedB *prep = nullptr;
    {
        auto it = g_prepared.find((const void *)d.B);
        if (it != g_prepared.end() && it->second.groups == d.groups && it->second.b32 == (d.b32 ? 1 : 0) && it->second.N == d.N && it->second.K == d.K)
            prep = &it->second;
    }
    if (prep) { p.grp_b = prep->table; p.b_nsub = prep->nsub; p.b_ksteps = prep->ksteps; }
    int na = g_cache.lookup(key_a), nb = prep ? prep->nb : g_cache.lookup(key_b);
    bool na_guessed = false, informed = nb != 0;
    if (!na) {
        auto it = g_cache.partner_a.find(key_b);
        na = it != g_cache.partner_a.end() ? it->second : 5;
        informed = informed && it != g_cache.partner_a.end();
        na_guessed = true;
    }
    if (!nb) nb = 5;
    // Both digit counts come from what these weights met before: speculate, do not wait.  A guarded launch of the
    // 16-row kernels follows on the stream (they guess nothing and take every operand); its workgroups return at once
    // unless the verdict is bad, in which case they compute every output again.  What the kernels saw travels to pinned
    // host memory behind an event and reaches the cache at a later call.  Otherwise (first sight of the weights, no
    // free slot) the verdict is read back before the call returns, as it used to be for every grouped launch.
    PendingRange *slot = nullptr;
    if (informed && g_cache.pinned && !g_switches.sync_verdict) {
        PendingRange &s = g_cache.pending[g_cache.pending_head];
        if (!s.busy && s.ev) slot = &s;
    }

    for (int attempt = 0; attempt < 3; attempt++) {
        const Instance *inst = nullptr;
        for (int tries = 0; tries < 2 && !inst; tries++) {
            inst = pick_instance(na, nb, d.b32 != 0 && !prep, true, 16, prep ? prep->nb : 0, prep ? kB64GroupBPlanes : -1, prep ? prep->kk : 1);
            if (!inst && prep && (inst = pick_instance(na, nb, d.b32 != 0, true)) != nullptr) {
                // no kernel with exactly the planes' digit count covers A: this call splits the original weights
                prep = nullptr;
                p.grp_b = d.B;
            }
            // a guess taken over from other activations that no 32-row kernel covers: try the widest they have (the
            // digit check settles it, and the guess would otherwise never be replaced)
            if (!inst && na_guessed && na > 5) na = 5; else break;
        }
        if (!inst) return 1;
        MfmaKernel fn = inst->fn[prep ? kB64GroupBPlanes : (d.b32 ? kB32Group : kB64Group)];
        if (!fn) return 1;
        // int32 weights, whole steps, rows of A on 16-byte boundaries, sixteen digit pairs or more: the form that streams the
        // weights through LDS rings.  (Measured on 256 experts, one box, streamed against general: (3,4) digits 5.64
        // against 5.86 TB/s at K = 7168 and level at K = 2048; (4,4) level at K = 7168 and 5.08 against 3.15 at K = 2048;
        // (5,5) 4.18 against 3.87.  ZK_STREAM32_MIN_PAIRS moves the limit.)
        size_t stream_lds = 0;
        if (d.b32 && !prep && !g_switches.no_stream32 && d.K % 32 == 0 && (((uintptr_t)d.A | (uintptr_t)(d.lda * 8)) & 15) == 0 && inst->bn == 256 &&
            inst->na * inst->nb >= g_switches.stream32_min_pairs) {
            MfmaKernel sfn = stream32_grouped_kernel(inst->na, inst->nb, &stream_lds);
            if (!sfn) sfn = stream32_grouped_kernel_wide(inst->na, inst->nb, &stream_lds);
            if (sfn) fn = sfn; else stream_lds = 0;
        }
        const long pairs = inst->na < inst->nb ? inst->na : inst->nb;
        const int ksteps = (d.K + 31) / 32;
        if (pairs * ksteps * 32 * 16384 > 0x7FFFFFFFL) return 1;
        p.tiles_n = (d.N + inst->bn - 1) / inst->bn;
        const long max_mtiles = (long)d.rows / 32 + d.groups;
        const long blocks = (max_mtiles + 7) / 8 * 8 * p.tiles_n;       // (whole rounds of the 8 XCDs: see the kernels' tile order)
        if (blocks > 0x7FFFFFFFL / 8) return 1;
        p.main_tiles = (int)blocks;
        if (const Outcome got = grow(g_cache.wg, g_cache.wg_count, (size_t)blocks * 4, "range slots")) return got;
        p.wg_range = g_cache.wg;
        const size_t lds = stream_lds ? stream_lds : 2 * (size_t)inst->kk * ((inst->bm / 32) * inst->na + (inst->bn / 32) * inst->nb) * 1024 + 9 * 1024 + 16;
        static std::set<const void *> lds_raised;
        if (lds > 64 * 1024 && !lds_raised.count((const void *)fn)) {
            if (hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
                set_error(kLaunchFailure, "grouped gemm: cannot raise the LDS limit to %zu bytes", lds);
                return -1;
            }
            lds_raised.insert((const void *)fn);
        }
        fn<<<dim3((unsigned)blocks), dim3((unsigned)inst->threads), lds, 0>>>(p);
        if (stream_lds) g_streamed_calls++;
        g_last_pairs = kept_pairs_before(inst->na, inst->nb, inst->dmax, inst->na, 0);
        g_last_prepared = prep ? 1 : 0;
        {
            const hipError_t err = hipGetLastError();
            if (err != hipSuccess) {
                set_error(kLaunchFailure, "grouped gemm: launch failed (%s; digits %d,%d, %ld workgroups)", hipGetErrorString(err), inst->na, inst->nb, blocks);
                return -1;
            }
        }
        const FoldArgs fold = make_fold(nullptr, 0, g_cache.wg, blocks, p.range, inst->na, inst->nb, slot ? slot->host : nullptr);
        range_fold_kernel<<<dim3((unsigned)fold.parts), 256, 0, 0>>>(fold);
        if (slot) {
            const int rc = gemm_rows16_grouped(d, p.range + 4);
            if (rc < 0) return -1;
            if (rc == 0) {
                *limbs_a = inst->na;
                *limbs_b = inst->nb;
                if (hipEventRecord(slot->ev, 0) == hipSuccess) {
                    slot->key_a = key_a;
                    slot->key_b = key_b;
                    slot->nb_fixed = prep ? prep->nb : 0;
                    slot->busy = true;
                    g_cache.pending_head = (g_cache.pending_head + 1) % kPendingSlots;
                } else {
                    (void)hipGetLastError();
                }
                return 0;
            }
            slot = nullptr;         // the 16-row kernels do not take this product: wait for the verdict after all
        }
        int64_t r[4];
        if (!read_range(p.range, r)) { set_error(kLaunchFailure, "grouped gemm: range readback failed"); return -1; }
        const int need_a = limbs_needed(r[0], r[1]), need_b = prep ? prep->nb : limbs_needed(r[2], r[3]);
        g_cache.store_pair(key_a, need_a, key_b, need_b);
        *limbs_a = inst->na;
        *limbs_b = inst->nb;
        if (need_a <= inst->na && need_b <= inst->nb) return 0;
        na = need_a;
        nb = need_b;
        na_guessed = false;
    }
    set_error(kLaunchFailure, "grouped gemm: digit count did not settle");
    return -1;
}

}  // namespace zk
