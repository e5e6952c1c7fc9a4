// Expert routing of the MoE gate in exact integers: one wavefront per token.
//
// Restates the tensor ops of Gate.forward (inference/model.py:1143-1208) on the sigmoid scores the gate's kernel
// part produced: add the bias, score every group of experts by the sum of its two largest biased scores (by its
// maximum when there is no bias), keep the `topk_groups` best groups, take the `topk` largest biased scores among
// the kept groups (the others count as -2^42), gather the UNBIASED scores of the winners, and normalise them:
// w = floor(floor(w * 2^23 / sum w) * 5 / 2).  Winners come out in descending order of biased score.
// Where values tie, torch.topk leaves the order to its implementation; here the lower index wins.
#include "common.h"
#include "../../include/int64gemm.h"

namespace zk {

struct Best { int64_t v; int idx; };

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

// EPL elements per lane, element e = lane * EPL + j.
template <int EPL>
__global__ __launch_bounds__(256) void gate_route_kernel(const int64_t *__restrict__ scores, const int32_t *__restrict__ bias,
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

}  // namespace zk

extern "C" void gate_route_q23(const int64_t *scores, const int32_t *bias, int64_t *weights, int64_t *indices,
                               int64_t *raw_weights, int T, int E, int n_groups, int topk_groups, int topk)
{
    const char *name = "gate_route_q23";
    if (T < 0 || E <= 0 || n_groups <= 0 || topk_groups <= 0 || topk <= 0) { zk::set_error(zk::kBadArgument, "%s: bad dimension", name); return; }
    if (T == 0) return;
    if (!scores || !weights || !indices) { zk::set_error(zk::kBadArgument, "%s: null pointer", name); return; }
    if (E > 1024) { zk::set_error(zk::kUnsupportedSize, "%s: more than 1024 experts", name); return; }
    if (n_groups > 64 || E % n_groups != 0 || topk_groups > n_groups || topk > 64 || topk > E) {
        zk::set_error(zk::kBadArgument, "%s: groups must divide the experts (at most 64), topk at most 64 and E", name);
        return;
    }
    const dim3 grid((unsigned)((T + 3) / 4)), block(256);
#define ZK_GATE(EPL) zk::gate_route_kernel<EPL><<<grid, block, 0, 0>>>(scores, bias, weights, indices, raw_weights, T, E, n_groups, topk_groups, topk)
    if (E <= 64) ZK_GATE(1);
    else if (E <= 128) ZK_GATE(2);
    else if (E <= 256) ZK_GATE(4);
    else if (E <= 512) ZK_GATE(8);
    else ZK_GATE(16);
#undef ZK_GATE
    zk::check_launch(name);
}
