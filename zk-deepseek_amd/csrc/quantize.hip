// Float checkpoint -> fixed-point weights on the device.
//
// The reference builds its integer weights in inference/convert2.py with tensor ops around a Triton kernel:
//   fp8 weights:   w = weight_dequant(w_fp8, scale)                     (inference/kernel.py:67-117: e4m3 value times
//                  the float32 scale of its 128x128 block, stored in the default dtype, bfloat16: convert2.py:185)
//                  w_int = (w.to(float32) * 2^k).round().to(int32)      (convert2.py:144-147, 308-311, 325-328, ...)
//   bf16 params:   p_int = (p.to(float32) * 2^k).round().to(int32|int64) (convert2.py:250-262, 290-295, 353-359)
// Each step is one IEEE operation, restated here per element: exact fp8 -> float32, one float32 multiply (round to
// nearest even), float32 -> bfloat16 (round to nearest even), an exact power-of-two scaling, round half to even, and
// the float -> integer conversion of the device the reference runs on (saturating, NaN -> 0).
// One pass: 1 byte read and 4 written per fp8 weight, instead of six tensor-sized round trips.
#include "common.h"
#include "../../include/int64gemm.h"

namespace zk {

constexpr int kScaleBlock = 128;      // weight_dequant's block_size default (inference/kernel.py:96)

// OCP e4m3fn byte `sel` of a packed word -> float32, exact (1 sign, 4 exponent with bias 7, 3 mantissa bits; no
// infinities, S.1111.111 is NaN): gfx950's own conversion instruction
template <int SEL>
__device__ __forceinline__ float e4m3fn_to_f32(uint32_t packed)
{
    return __builtin_amdgcn_cvt_f32_fp8((int)packed, SEL);
}

// float32 -> bfloat16 -> float32, round to nearest even (NaN stays NaN): the hardware conversion, as a cast
__device__ __forceinline__ float round_to_bf16(float v)
{
    return (float)(__bf16)v;
}

// round half to even, then convert as the reference's device does: saturate, NaN -> 0.  That is what v_cvt_i32_f32
// does on its own; the instruction is named because a C++ cast is undefined outside the int32 range.
__device__ __forceinline__ int32_t round_to_i32(float z)
{
    int32_t o;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(o) : "v"(rintf(z)));
    return o;
}

__device__ __forceinline__ int64_t round_to_i64(float z)
{
    const float r = rintf(z);
    if (!(r == r)) return 0;
    if (r >= 9223372036854775808.0f) return INT64_MAX;
    if (r <= -9223372036854775808.0f) return INT64_MIN;
    return (int64_t)r;
}

typedef int v4i_q __attribute__((ext_vector_type(4)));

// Four consecutive weights of a row per thread and round (cols % 4 == 0, aligned pointers): a 4-byte load and a 16-byte
// store, adjacent lanes on adjacent pieces so that both are contiguous over the wave; four rounds in flight per thread.
// A 128-wide scale block covers whole 4-element pieces, so one scale serves a piece.
__global__ __launch_bounds__(256) void fp8_to_int32_vec_kernel(const uint8_t *__restrict__ w, const float *__restrict__ scale,
                                                               int32_t *__restrict__ out, int rows, int pieces_per_row,
                                                               int scale_cols, float mult)
{
    // blockIdx.y walks the rows, blockIdx.x the 1024-piece stretches of a row: no division anywhere
    for (int row = blockIdx.y; row < rows; row += gridDim.y) {
        const float *srow = scale + (long)(row / kScaleBlock) * scale_cols;
        const uint32_t *wrow = reinterpret_cast<const uint32_t *>(w) + (long)row * pieces_per_row;
        v4i_q *orow = reinterpret_cast<v4i_q *>(out) + (long)row * pieces_per_row;
        for (int base = blockIdx.x * 1024; base < pieces_per_row; base += gridDim.x * 1024) {
            uint32_t in[4];
            float s[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int pc = base + u * 256 + threadIdx.x;
                if (pc < pieces_per_row) {
                    in[u] = __builtin_nontemporal_load(wrow + pc);
                    s[u] = srow[pc / (kScaleBlock / 4)];
                }
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int pc = base + u * 256 + threadIdx.x;
                if (pc < pieces_per_row) {
                    v4i_q o;
                    o[0] = round_to_i32(round_to_bf16(e4m3fn_to_f32<0>(in[u]) * s[u]) * mult);
                    o[1] = round_to_i32(round_to_bf16(e4m3fn_to_f32<1>(in[u]) * s[u]) * mult);
                    o[2] = round_to_i32(round_to_bf16(e4m3fn_to_f32<2>(in[u]) * s[u]) * mult);
                    o[3] = round_to_i32(round_to_bf16(e4m3fn_to_f32<3>(in[u]) * s[u]) * mult);
                    __builtin_nontemporal_store(o, orow + pc);
                }
            }
        }
    }
}

__global__ __launch_bounds__(256) void fp8_to_int32_kernel(const uint8_t *__restrict__ w, const float *__restrict__ scale,
                                                           int32_t *__restrict__ out, long n, int cols, int scale_cols, float mult)
{
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
        const long row = i / cols;
        const int col = (int)(i - row * cols);
        const float s = scale[(row / kScaleBlock) * scale_cols + col / kScaleBlock];
        out[i] = round_to_i32(round_to_bf16(e4m3fn_to_f32<0>(w[i]) * s) * mult);
    }
}

template <typename OT>
__global__ __launch_bounds__(256) void bf16_round_kernel(const uint16_t *__restrict__ in, OT *__restrict__ out, long n, float mult)
{
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
        const float z = __uint_as_float((uint32_t)in[i] << 16) * mult;
        if (sizeof(OT) == 4) out[i] = (OT)round_to_i32(z);
        else out[i] = (OT)round_to_i64(z);
    }
}

static unsigned grid_for(long items)
{
    const long blocks = (items + 255) / 256;
    return (unsigned)(blocks < 1 ? 1 : (blocks > 65536 * 4 ? 65536 * 4 : blocks));
}

// 2^k as a float32, the scalar the reference multiplies by; k in [0,127] keeps it finite
static bool pow2_ok(const char *name, int k, float *mult)
{
    if (k < 0 || k > 127) { set_error(kBadArgument, "%s: exponent %d outside 0..127", name, k); return false; }
    *mult = ldexpf(1.0f, k);
    return true;
}

template <typename OT>
static void launch_bf16_round(const char *name, const uint16_t *in, OT *out, long n, int k)
{
    float mult;
    if (n < 0) { set_error(kBadArgument, "%s: negative size", name); return; }
    if (!pow2_ok(name, k, &mult) || n == 0) return;
    if (!in || !out) { set_error(kBadArgument, "%s: null pointer", name); return; }
    bf16_round_kernel<OT><<<dim3(grid_for(n)), dim3(256), 0, 0>>>(in, out, n, mult);
    check_launch(name);
}

}  // namespace zk

extern "C" {

void fp8_block_scaled_to_int32(const uint8_t *w, const float *scale, int32_t *out, int rows, int cols, int k)
{
    const char *name = "fp8_block_scaled_to_int32";
    float mult;
    if (rows < 0 || cols < 0) { zk::set_error(zk::kBadArgument, "%s: negative dimension", name); return; }
    if (!zk::pow2_ok(name, k, &mult) || (long)rows * cols == 0) return;
    if (!w || !scale || !out) { zk::set_error(zk::kBadArgument, "%s: null pointer", name); return; }
    const int scale_cols = (cols + zk::kScaleBlock - 1) / zk::kScaleBlock;
    const long n = (long)rows * cols;
    if (cols % 4 == 0 && ((uintptr_t)w & 3) == 0 && ((uintptr_t)out & 15) == 0) {
        const int ppr = cols / 4;
        const dim3 grid((unsigned)((ppr + 4095) / 4096), (unsigned)(rows < 65535 ? rows : 65535));     // a workgroup walks up to 4 stretches
        zk::fp8_to_int32_vec_kernel<<<grid, dim3(256), 0, 0>>>(w, scale, out, rows, ppr, scale_cols, mult);
    } else {
        zk::fp8_to_int32_kernel<<<dim3(zk::grid_for(n)), dim3(256), 0, 0>>>(w, scale, out, n, cols, scale_cols, mult);
    }
    zk::check_launch(name);
}

void bf16_scaled_round_to_int32(const uint16_t *in, int32_t *out, long n, int k)
{
    zk::launch_bf16_round<int32_t>("bf16_scaled_round_to_int32", in, out, n, k);
}

void bf16_scaled_round_to_int64(const uint16_t *in, int64_t *out, long n, int k)
{
    zk::launch_bf16_round<int64_t>("bf16_scaled_round_to_int64", in, out, n, k);
}

}  // extern "C"
