// Measurement helper: what the i8 matrix pipe sustains on this device, for the roofline of the MFMA GEMM path.
//
// The figure depends on the operand values: the device is power managed, and MFMAs fed with bytes that toggle
// at random run markedly slower than the same instruction stream fed with zeros.  The balanced base-256 digits
// of real operands are random bytes, so both figures are reported and the random one is the honest ceiling.
#include "common.h"
#include "../../include/int64gemm.h"

namespace zk {

typedef int pv4i __attribute__((ext_vector_type(4)));
typedef int pv16i __attribute__((ext_vector_type(16)));

__device__ __forceinline__ unsigned probe_hash(unsigned x)
{
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}

// 8 waves per workgroup, 10 accumulator tiles per wave (two 32x32 tiles x five digit diagonals, as in the narrow
// GEMM tile), 18 MFMAs per wave and step.  WITH_LDS: the nine operand fragments of a step are read from LDS
// and a barrier closes the step, as in the GEMM; otherwise the operands stay in registers.
template <bool WITH_LDS>
__global__ __launch_bounds__(512) void probe_mfma_kernel(int steps, int random_data, int *sink)
{
    __shared__ __attribute__((aligned(16))) unsigned char sm[65536];
    for (int i = threadIdx.x; i < 16384; i += 512)
        reinterpret_cast<unsigned *>(sm)[i] = random_data ? probe_hash(i * 7919u + blockIdx.x) : 0u;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    pv16i acc[10];
#pragma unroll
    for (int i = 0; i < 10; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0;
    pv4i f[9];
#pragma unroll
    for (int j = 0; j < 9; j++) f[j] = *reinterpret_cast<const pv4i *>(sm + ((wave * 9 + j) & 63) * 1024 + lane * 16);
    for (int it = 0; it < steps; it++) {
        if (WITH_LDS) {
#pragma unroll
            for (int j = 0; j < 9; j++) f[j] = *reinterpret_cast<const pv4i *>(sm + ((wave * 9 + j + it) & 63) * 1024 + lane * 16);
        }
#pragma unroll
        for (int i = 0; i < 3; i++)
#pragma unroll
            for (int j = 0; j < 3; j++) {
                acc[i + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f[i], f[6 + j], acc[i + j], 0, 0, 0);
                acc[5 + i + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f[3 + i], f[6 + j], acc[5 + i + j], 0, 0, 0);
            }
        if (WITH_LDS) __syncthreads();
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 10; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) s += acc[i][r];
    if (s == 0x7f3a91c5 && steps < 0) sink[0] = s;       // never true: keeps the accumulators alive
}

// The smallest thing a call made of two dependent launches can be: every workgroup of the first kernel stores 16 bytes,
// every thread group of the second loads them and stores one word.  What this pair costs per repetition, back to back on
// the null stream, is what the launches themselves cost a split-K call (one kernel that streams, one that adds up).
__global__ __launch_bounds__(256) void probe_pair_first(unsigned long long *buf)
{
    if (threadIdx.x == 0) {
        buf[2 * blockIdx.x] = blockIdx.x;
        buf[2 * blockIdx.x + 1] = ~(unsigned long long)blockIdx.x;
    }
}

__global__ __launch_bounds__(256) void probe_pair_second(const unsigned long long *buf, unsigned long long *out, int n)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = buf[2 * i] + buf[2 * i + 1];
}

}  // namespace zk

namespace zk {

// What the device takes in streaming stores alone (nothing read): every thread writes 16-byte pieces, non-temporal, the
// grid striding over the buffer.  The ceiling of a kernel whose traffic is mostly writes (the fp8 checkpoint quantiser
// writes four bytes per byte read).
__global__ __launch_bounds__(256) void probe_store_kernel(pv4i *out, long pieces, int seed)
{
    const pv4i v = { seed, seed + 1, seed + 2, seed + 3 };
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < pieces; i += (long)gridDim.x * 256) __builtin_nontemporal_store(v, out + i);
}

}  // namespace zk

extern "C" double zk_probe_store_gbps(long bytes, int reps)
{
    if (bytes < 4096 || reps <= 0) { zk::set_error(zk::kBadArgument, "zk_probe_store_gbps: bad argument"); return 0.0; }
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    zk::pv4i *buf = nullptr;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    double gbps = 0.0;
    const long pieces = bytes / 16;
    if (hipMalloc(&buf, (size_t)pieces * 16) == hipSuccess && hipEventCreate(&t0) == hipSuccess && hipEventCreate(&t1) == hipSuccess) {
        for (int r = 0; r < 3; r++) zk::probe_store_kernel<<<dim3((unsigned)(cus * 8)), dim3(256), 0, 0>>>(buf, pieces, r);
        (void)hipEventRecord(t0, 0);
        for (int r = 0; r < reps; r++) zk::probe_store_kernel<<<dim3((unsigned)(cus * 8)), dim3(256), 0, 0>>>(buf, pieces, r);
        (void)hipEventRecord(t1, 0);
        float ms = 0.f;
        if (hipEventSynchronize(t1) == hipSuccess && hipEventElapsedTime(&ms, t0, t1) == hipSuccess && ms > 0.f)
            gbps = (double)pieces * 16.0 * reps / (ms * 1e-3) / 1e9;
    }
    if (hipGetLastError() != hipSuccess || gbps == 0.0) zk::set_error(zk::kLaunchFailure, "zk_probe_store_gbps: measurement failed");
    if (t0) (void)hipEventDestroy(t0);
    if (t1) (void)hipEventDestroy(t1);
    if (buf) (void)hipFree(buf);
    return gbps;
}

extern "C" double zk_probe_launch_pair_us(int workgroups, int reps)
{
    if (workgroups <= 0 || workgroups > 65536 || reps <= 0) { zk::set_error(zk::kBadArgument, "zk_probe_launch_pair_us: bad argument"); return 0.0; }
    unsigned long long *buf = nullptr;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    double us = 0.0;
    if (hipMalloc(&buf, (size_t)workgroups * 3 * sizeof(unsigned long long)) == hipSuccess && hipEventCreate(&t0) == hipSuccess &&
        hipEventCreate(&t1) == hipSuccess) {
        auto pair = [&] {
            zk::probe_pair_first<<<dim3((unsigned)workgroups), dim3(256), 0, 0>>>(buf);
            zk::probe_pair_second<<<dim3((unsigned)((workgroups + 255) / 256)), dim3(256), 0, 0>>>(buf, buf + 2 * (size_t)workgroups, workgroups);
        };
        for (int r = 0; r < 10; r++) pair();
        (void)hipEventRecord(t0, 0);
        for (int r = 0; r < reps; r++) pair();
        (void)hipEventRecord(t1, 0);
        float ms = 0.f;
        if (hipEventSynchronize(t1) == hipSuccess && hipEventElapsedTime(&ms, t0, t1) == hipSuccess && ms > 0.f) us = (double)ms * 1e3 / reps;
    }
    if (hipGetLastError() != hipSuccess || us == 0.0) zk::set_error(zk::kLaunchFailure, "zk_probe_launch_pair_us: measurement failed");
    if (t0) (void)hipEventDestroy(t0);
    if (t1) (void)hipEventDestroy(t1);
    if (buf) (void)hipFree(buf);
    return us;
}

extern "C" double zk_probe_mfma_i8_tops(int with_lds, int random_data, int steps)
{
    if (steps <= 0) { zk::set_error(zk::kBadArgument, "zk_probe_mfma_i8_tops: steps must be positive"); return 0.0; }
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
        zk::set_error(zk::kLaunchFailure, "zk_probe_mfma_i8_tops: cannot query the device");
        return 0.0;
    }
    int *sink = nullptr;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    double tops = 0.0;
    if (hipMalloc(&sink, sizeof(int)) == hipSuccess && hipEventCreate(&t0) == hipSuccess && hipEventCreate(&t1) == hipSuccess) {
        auto launch = [&] {
            if (with_lds) zk::probe_mfma_kernel<true><<<dim3(cus), dim3(512), 0, 0>>>(steps, random_data, sink);
            else zk::probe_mfma_kernel<false><<<dim3(cus), dim3(512), 0, 0>>>(steps, random_data, sink);
        };
        launch();                                            // warm-up
        const int reps = 5;
        (void)hipEventRecord(t0, 0);
        for (int r = 0; r < reps; r++) launch();
        (void)hipEventRecord(t1, 0);
        float ms = 0.f;
        if (hipEventSynchronize(t1) == hipSuccess && hipEventElapsedTime(&ms, t0, t1) == hipSuccess && ms > 0.f) {
            const double macs = (double)cus * 8 * steps * 18 * 32768.0 * reps;
            tops = 2.0 * macs / (ms * 1e-3) / 1e12;
        }
    }
    if (hipGetLastError() != hipSuccess || tops == 0.0) zk::set_error(zk::kLaunchFailure, "zk_probe_mfma_i8_tops: measurement failed");
    if (t0) (void)hipEventDestroy(t0);
    if (t1) (void)hipEventDestroy(t1);
    if (sink) (void)hipFree(sink);
    return tops;
}
