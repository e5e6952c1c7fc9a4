// Expert routing of the MoE gate in exact integers: one wavefront per token.
//
// Restates the tensor ops of Gate.forward (inference/model.py:1143-1208) on the sigmoid scores the gate's kernel
// part produced: add the bias, score every group of experts by the sum of its two largest biased scores (by its
// maximum when there is no bias), keep the `topk_groups` best groups, take the `topk` largest biased scores among
// the kept groups (the others count as -2^42), gather the UNBIASED scores of the winners, and normalise them:
// w = floor(floor(w * 2^23 / sum w) * 5 / 2).  Winners come out in descending order of biased score.
// Where values tie, torch.topk leaves the order to its implementation; here the lower index wins.
#include "common.h"
#include "act_one.h"
#include "../../include/int64gemm.h"

namespace zk {

struct Best { int64_t v; int idx; };
struct __attribute__((aligned(16))) i64x2g { int64_t x, y; };

// larger value wins; on equal values the lower index
__device__ __forceinline__ Best better(Best a, Best b)
{
    const bool take_b = b.v > a.v || (b.v == a.v && b.idx < a.idx);
    return take_b ? b : a;
}

__device__ __forceinline__ Best wave_best(Best x)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        Best o;
        o.v = __shfl_xor(x.v, off, kWave);
        o.idx = __shfl_xor(x.idx, off, kWave);
        x = better(x, o);
    }
    return x;
}

__device__ __forceinline__ int64_t floordiv64(int64_t a, int64_t b)
{
    if (b == 0) return 0;
    int64_t q = tdiv64(a, b);
    if ((a % b != 0) && ((a < 0) != (b < 0))) q--;
    return q;
}

constexpr int64_t kMasked = -((int64_t)1 << 42);
constexpr int kNone = 0x7FFFFFFF;

// EPL elements per lane, element e = lane * EPL + j.  FUSED: `scores` holds the gate's logits; their sigmoid (Q23, table
// `lut`) is taken here and stored to `sig` when that is not null.
template <int EPL, bool FUSED>
__global__ __launch_bounds__(256) void gate_route_kernel(const int64_t *__restrict__ scores, const int64_t *__restrict__ lut,
                                                         int64_t *__restrict__ sig, const int32_t *__restrict__ bias,
                                                         int64_t *__restrict__ weights, int64_t *__restrict__ indices,
                                                         int64_t *__restrict__ raw, int T, int E, int n_groups,
                                                         int topk_groups, int topk)
{
    const int lane = threadIdx.x & 63;
    const long tok = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tok >= T) return;
    const int64_t *row = scores + tok * E;
    int64_t orig[EPL], s[EPL];
    bool live[EPL];
#pragma unroll
    for (int j = 0; j < EPL; j++) {
        const int e = lane * EPL + j;
        live[j] = e < E;
        orig[j] = live[j] ? row[e] : 0;
        if (FUSED && live[j]) {
            orig[j] = act_one<23, true>(orig[j], lut);
            if (sig) sig[tok * E + e] = orig[j];
        }
        s[j] = live[j] ? (int64_t)((uint64_t)orig[j] + (uint64_t)(int64_t)(bias ? bias[e] : 0)) : 0;
    }

    if (n_groups > 1) {
        // lane g ends up holding the score of group g
        const int gsize = E / n_groups;
        int grp[EPL];                                     // group of every element (one division each, not one per test)
#pragma unroll
        for (int j = 0; j < EPL; j++) grp[j] = live[j] ? (lane * EPL + j) / gsize : -1;
        int64_t my_group_score = 0;
        for (int g = 0; g < n_groups; g++) {
            Best b1 = { INT64_MIN, kNone };
#pragma unroll
            for (int j = 0; j < EPL; j++) {
                const int e = lane * EPL + j;
                if (grp[j] == g) b1 = better(b1, Best{ s[j], e });
            }
            b1 = wave_best(b1);
            int64_t gs = b1.v;
            if (bias) {                                   // top-2 sum: the best of the rest of the group
                Best b2 = { INT64_MIN, kNone };
#pragma unroll
                for (int j = 0; j < EPL; j++) {
                    const int e = lane * EPL + j;
                    if (grp[j] == g && e != b1.idx) b2 = better(b2, Best{ s[j], e });
                }
                b2 = wave_best(b2);
                gs = (int64_t)((uint64_t)gs + (uint64_t)(b2.idx == kNone ? 0 : b2.v));
            }
            if (lane == g) my_group_score = gs;
        }
        // rank of group `lane` among the groups (ties: the lower group first), then every element asks its group
        int rank = 0;
        for (int h = 0; h < n_groups; h++) {
            const int64_t o = __shfl(my_group_score, h, kWave);
            if (o > my_group_score || (o == my_group_score && h < lane)) rank++;
        }
        const int keep = (lane < n_groups && rank < topk_groups) ? 1 : 0;
#pragma unroll
        for (int j = 0; j < EPL; j++) {
            const int kept = __shfl(keep, live[j] ? grp[j] : 0, kWave);
            if (live[j] && !kept) s[j] = kMasked;
        }
    }

    // the topk largest, one wave-wide arg-max per winner
    int64_t wsum = 0, my_w = 0;                     // lane i < topk keeps the unbiased score of winner i
    int my_idx = 0;
    bool taken[EPL];
#pragma unroll
    for (int j = 0; j < EPL; j++) taken[j] = !live[j];
    for (int i = 0; i < topk; i++) {
        Best b = { INT64_MIN, kNone };
#pragma unroll
        for (int j = 0; j < EPL; j++)
            if (!taken[j]) b = better(b, Best{ s[j], lane * EPL + j });
        b = wave_best(b);
        int64_t w = 0;
#pragma unroll
        for (int j = 0; j < EPL; j++)
            if (lane * EPL + j == b.idx) { taken[j] = true; w = orig[j]; }
        w = __shfl(w, b.idx / EPL, kWave);
        wsum = (int64_t)((uint64_t)wsum + (uint64_t)w);
        if (lane == i) { my_w = w; my_idx = b.idx; }
    }
    if (lane < topk) {
        if (raw) raw[tok * topk + lane] = my_w;
        int64_t w = floordiv64((int64_t)((uint64_t)my_w << 23), wsum);      // (w * 2^23) // sum  (model.py:1203)
        w = floordiv64((int64_t)((uint64_t)w * 5ull), 2);                    // w * 5 // 2         (model.py:1208)
        weights[tok * topk + lane] = w;
        indices[tok * topk + lane] = my_idx;
    }
}

// The same routing with the experts of a token spread over LT = NG * LPG lanes: lane l holds the GS consecutive scores
// from l * GS on in registers, LPG neighbouring lanes make up a group.  The groups' two best, the masking and most of the
// arg-max over a token's experts (GS comparisons per lane, log2(LT) exchanges) stay inside a lane; the wave-wide form
// above pays six exchanges per group and per winner.  LPG = 1 gives the most tokens per wavefront (throughput when
// there are many tokens), LPG = 4 the shorter chain of dependent work per token (latency when there are few).
template <int GS, int LPG, int NG, bool FUSED>
__global__ __launch_bounds__(256) void gate_route_groups_kernel(const int64_t *__restrict__ scores, const int64_t *__restrict__ lut,
                                                                int64_t *__restrict__ sig, const int32_t *__restrict__ bias,
                                                                int64_t *__restrict__ weights, int64_t *__restrict__ indices,
                                                                int64_t *__restrict__ raw, int T, int topk_groups, int topk)
{
    constexpr int LT = NG * LPG, E = GS * LT, kTokens = 64 / LT;
    static_assert(LT <= 64 && GS % 2 == 0, "a token fits a wavefront; 16-byte loads");
    const int lane = threadIdx.x & 63, l = lane % LT, g = l / LPG, first = lane - l;
    const long tok_raw = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * kTokens + lane / LT;
    const bool tok_live = tok_raw < T;
    const long tok = tok_live ? tok_raw : T - 1;          // lanes past the end walk the last token along and store nothing
    const int64_t *row = scores + tok * E + l * GS;
    int64_t s[GS];
#pragma unroll
    for (int j = 0; j < GS; j += 2) {
        const i64x2g v = *reinterpret_cast<const i64x2g *>(row + j);
        s[j] = v.x;
        s[j + 1] = v.y;
    }
    if (FUSED) {
#pragma unroll
        for (int j = 0; j < GS; j++) s[j] = act_one<23, true>(s[j], lut);
        if (sig && tok_live) {
#pragma unroll
            for (int j = 0; j < GS; j += 2) *reinterpret_cast<i64x2g *>(sig + tok * E + l * GS + j) = i64x2g{ s[j], s[j + 1] };
        }
    }
    if (bias) {
#pragma unroll
        for (int j = 0; j < GS; j++) s[j] = (int64_t)((uint64_t)s[j] + (uint64_t)(int64_t)bias[l * GS + j]);
    }

    // the group's score: its two largest biased scores (its largest without bias); then the group's rank
    int64_t b1 = s[0], b2 = INT64_MIN;
#pragma unroll
    for (int j = 1; j < GS; j++) {
        const bool first_j = s[j] > b1;
        const int64_t lower = first_j ? b1 : s[j];
        b1 = first_j ? s[j] : b1;
        b2 = lower > b2 ? lower : b2;
    }
#pragma unroll
    for (int off = LPG / 2; off > 0; off >>= 1) {          // the two best of both halves: the larger first, then the best of the rest
        const int64_t o1 = __shfl_xor(b1, off, kWave), o2 = __shfl_xor(b2, off, kWave);
        const int64_t lo = b1 > o1 ? o1 : b1, rest = b2 > o2 ? b2 : o2;
        b1 = b1 > o1 ? b1 : o1;
        b2 = lo > rest ? lo : rest;
    }
    const int64_t gs = bias ? (int64_t)((uint64_t)b1 + (uint64_t)b2) : b1;
    int rank = 0;
#pragma unroll
    for (int h = 0; h < NG; h++) {
        const int64_t o = __shfl(gs, first + h * LPG, kWave);
        if (o > gs || (o == gs && h < g)) rank++;
    }
    const bool masked = rank >= topk_groups;               // every score of this lane counts as -2^42

    unsigned taken = 0;                                    // bit j: s[j] has won already
    int64_t wsum = 0;
    for (int i = 0; i < topk; i++) {
        // this lane's candidate: its largest score not taken (the lowest index on ties; a masked lane's scores all tie)
        Best b = { INT64_MIN, kNone };
#pragma unroll
        for (int j = 0; j < GS; j++) {
            const int64_t v = masked ? kMasked : s[j];
            if (!((taken >> j) & 1) && (b.idx == kNone || v > b.v)) b = Best{ v, l * GS + j };
        }
#pragma unroll
        for (int off = LT / 2; off > 0; off >>= 1) {
            Best o;
            o.v = __shfl_xor(b.v, off, kWave);
            o.idx = __shfl_xor(b.idx, off, kWave);
            b = better(b, o);
        }
        // the owner gives the winner's unbiased score
        int64_t w = 0;
        if (b.idx / GS == l) {
            const int jw = b.idx % GS;
            taken |= 1u << jw;
            int64_t sv = 0;
#pragma unroll
            for (int j = 0; j < GS; j++) sv = j == jw ? s[j] : sv;
            w = bias ? (int64_t)((uint64_t)sv - (uint64_t)(int64_t)bias[b.idx]) : sv;
        }
        w = __shfl(w, first + b.idx / GS, kWave);
        wsum = (int64_t)((uint64_t)wsum + (uint64_t)w);
        if (l == i % LT && tok_live) {                     // parked in the outputs until the sum is known
            weights[tok * topk + i] = w;
            indices[tok * topk + i] = b.idx;
            if (raw) raw[tok * topk + i] = w;
        }
    }
    if (!tok_live) return;
    for (int i = l; i < topk; i += LT) {                   // (a lane reads back what it stored itself)
        int64_t w = floordiv64((int64_t)((uint64_t)weights[tok * topk + i] << 23), wsum);    // (w * 2^23) // sum  (model.py:1203)
        w = floordiv64((int64_t)((uint64_t)w * 5ull), 2);                                      // w * 5 // 2         (model.py:1208)
        weights[tok * topk + i] = w;
    }
}

template <bool FUSED>
static void gate_launch(const char *name, const int64_t *scores, const int64_t *lut, int64_t *sig, const int32_t *bias,
                        int64_t *weights, int64_t *indices, int64_t *raw, int T, int E, int n_groups, int topk_groups, int topk)
{
    if (T < 0 || E <= 0 || n_groups <= 0 || topk_groups <= 0 || topk <= 0) { set_error(kBadArgument, "%s: bad dimension", name); return; }
    if (T == 0) return;
    if (!scores || !weights || !indices || (FUSED && !lut)) { set_error(kBadArgument, "%s: null pointer", name); return; }
    if (E > 1024) { set_error(kUnsupportedSize, "%s: more than 1024 experts", name); return; }
    if (n_groups > 64 || E % n_groups != 0 || topk_groups > n_groups || topk > 64 || topk > E) {
        set_error(kBadArgument, "%s: groups must divide the experts (at most 64), topk at most 64 and E", name);
        return;
    }
    const int gsize = E / n_groups;
    const bool aligned = (((uintptr_t)scores | (uintptr_t)sig) & 15) == 0;
    const bool pow2 = (n_groups & (n_groups - 1)) == 0;
    if (aligned && pow2 && n_groups >= 2 && (gsize == 32 || gsize == 16 || gsize == 8) && n_groups <= 16) {
        // few tokens: four lanes per group (the chain of dependent work per token is what takes the time); many: one
        const bool spread = T <= 8192;
        const int per_wave = 64 / (n_groups * (spread ? 4 : 1));
        const dim3 grid((unsigned)((T + 4 * per_wave - 1) / (4 * per_wave))), block(256);
#define ZK_GATE_G(GS, LPG, NG) gate_route_groups_kernel<GS, LPG, NG, FUSED><<<grid, block, 0, 0>>>(scores, lut, sig, bias, weights, indices, raw, T, topk_groups, topk)
#define ZK_GATE_NG(GSIZE, NG) do { if (spread) ZK_GATE_G(GSIZE / 4, 4, NG); else ZK_GATE_G(GSIZE, 1, NG); } while (0)
#define ZK_GATE_GS(GSIZE) do { if (n_groups == 2) ZK_GATE_NG(GSIZE, 2); else if (n_groups == 4) ZK_GATE_NG(GSIZE, 4); \
                               else if (n_groups == 8) ZK_GATE_NG(GSIZE, 8); else ZK_GATE_NG(GSIZE, 16); } while (0)
        if (gsize == 32) ZK_GATE_GS(32);
        else if (gsize == 16) ZK_GATE_GS(16);
        else ZK_GATE_GS(8);
#undef ZK_GATE_GS
#undef ZK_GATE_NG
#undef ZK_GATE_G
        check_launch(name);
        return;
    }
    const dim3 grid((unsigned)((T + 3) / 4)), block(256);
#define ZK_GATE(EPL) gate_route_kernel<EPL, FUSED><<<grid, block, 0, 0>>>(scores, lut, sig, bias, weights, indices, raw, T, E, n_groups, topk_groups, topk)
    if (E <= 64) ZK_GATE(1);
    else if (E <= 128) ZK_GATE(2);
    else if (E <= 256) ZK_GATE(4);
    else if (E <= 512) ZK_GATE(8);
    else ZK_GATE(16);
#undef ZK_GATE
    check_launch(name);
}

}  // namespace zk

extern "C" void gate_route_q23(const int64_t *scores, const int32_t *bias, int64_t *weights, int64_t *indices,
                               int64_t *raw_weights, int T, int E, int n_groups, int topk_groups, int topk)
{
    zk::gate_launch<false>("gate_route_q23", scores, nullptr, nullptr, bias, weights, indices, raw_weights, T, E, n_groups, topk_groups, topk);
}

extern "C" void gate_sigmoid_route_q23(const int64_t *logits, const int64_t *lut, const int32_t *bias, int64_t *scores,
                                       int64_t *weights, int64_t *indices, int64_t *raw_weights, int T, int E,
                                       int n_groups, int topk_groups, int topk)
{
    zk::gate_launch<true>("gate_sigmoid_route_q23", logits, lut, scores, bias, weights, indices, raw_weights, T, E, n_groups, topk_groups, topk);
}
