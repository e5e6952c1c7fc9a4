// Shared declarations of libint64gemm.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __int128 i128;
typedef unsigned __int128 u128;

namespace zk {

enum ErrorCode { kOk = 0, kBadArgument = 1, kLaunchFailure = 2, kUnsupportedSize = 3 };

// Records the first error since zk_clear_error(); later ones are dropped so the cause is kept.
void set_error(int code, const char *fmt, ...);
// hipGetLastError() after a launch; records kLaunchFailure and returns false on failure.
bool check_launch(const char *what);

// Errors detected on the device: a pinned host flag per kind (null when pinned memory is not to be had) that a kernel
// sets to 1; zk_last_error() turns a set flag into a recorded error.
enum DeferredError { kDeferredMoeIndex = 0, kDeferredCount };
int *deferred_error_flag(int which);

// Device memory the library holds between calls (per module), and its release.
size_t gemm_mfma_workspace_bytes(size_t *prepared_bytes);
void gemm_mfma_release_workspace();
void gemm_mfma_reload_switches();
size_t act_workspace_bytes();
void act_release_workspace();

constexpr int kWave = 64;

// A pointer that came out of memory itself (an expert's matrix from the table of a grouped launch) could point anywhere
// as far as the compiler knows, and a load through it counts as an LDS access as well: every wait for LDS then waits
// for the weights under way.  Loads of operands name their address space: (const ZK_GLOBAL_MEM T *)ptr.
#define ZK_GLOBAL_MEM __attribute__((address_space(1)))

// ---- wave-level helpers --------------------------------------------------------------------
// 64-lane butterfly reductions.  Every lane ends up with the result.
__device__ __forceinline__ int64_t wave_max_i64(int64_t v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        int64_t o = __shfl_xor(v, off, kWave);
        v = o > v ? o : v;
    }
    return v;
}

__device__ __forceinline__ uint64_t wave_sum_u64(uint64_t v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += (uint64_t)__shfl_xor((long long)v, off, kWave);
    return v;
}

// ---- exact integer division helpers -----------------------------------------------------------
// C++ signed division with the two undefined corners fixed (b == 0 -> 0, INT64_MIN / -1 wraps).
__device__ __forceinline__ int64_t tdiv64(int64_t a, int64_t b)
{
    if (b == 0) return 0;
    if (b == -1) return (int64_t)(0 - (uint64_t)a);
    return a / b;
}

// floor(num / den) for 0 <= num < 2^53, 0 < den < 2^53 and quotient < 2^40, given inv = 1.0 / (double)den.
// The double estimate is within one of the quotient; the remainder test makes it exact.
__device__ __forceinline__ uint64_t udiv_by_inv(uint64_t num, uint64_t den, double inv)
{
    uint64_t q = (uint64_t)((double)num * inv);
    int64_t rem = (int64_t)(num - q * den);
    if (rem < 0) { q -= 1; rem += (int64_t)den; }
    if (rem >= (int64_t)den) q += 1;
    return q;
}

}  // namespace zk
