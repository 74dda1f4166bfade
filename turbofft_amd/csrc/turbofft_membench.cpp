// Streaming kernels of known traffic, for the measurements the FFT kernels are judged against:
// what a plain copy reaches on this device with 8-byte and with 16-byte lanes (the reason the fp32
// kernels move one float2 per lane), and what read-only and write-only sweeps reach.  Also the
// kernels of known size that rocprofv3's FETCH_SIZE / WRITE_SIZE counters can be scaled with.
// Measurement only: nothing here is used by turbofft_exec.  No counterpart in the reference, which
// quotes its bandwidth against the data sheet (readme.md).
#include <hip/hip_runtime.h>

#include "../../include/turbofft.h"

void tfft_set_error(const char* fmt, ...);   // turbofft_host.cpp

namespace {

typedef float v2 __attribute__((ext_vector_type(2)));
typedef float v4 __attribute__((ext_vector_type(4)));

// a block of 256 threads moves one contiguous tile of 256*U vectors: every load is issued before
// the first store, as in the FFT kernels; the lanes of a wavefront touch consecutive vectors
template <class V, int U>
__global__ __launch_bounds__(256) void tfft_mb_copy(const V* __restrict__ in, V* __restrict__ out) {
    const size_t base = (size_t)blockIdx.x * 256 * U + threadIdx.x;
    V r[U];
#pragma unroll
    for (int e = 0; e < U; ++e) r[e] = in[base + (size_t)e * 256];
#pragma unroll
    for (int e = 0; e < U; ++e) out[base + (size_t)e * 256] = r[e];
}

template <class V, int U>
__global__ __launch_bounds__(256) void tfft_mb_read(const V* __restrict__ in, float* __restrict__ sink) {
    const size_t base = (size_t)blockIdx.x * 256 * U + threadIdx.x;
    V r[U];
#pragma unroll
    for (int e = 0; e < U; ++e) r[e] = in[base + (size_t)e * 256];
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < U; ++e) acc += r[e].x;
    if (acc == 123456.789f) sink[0] = acc;       // keeps the loads alive, never true for the test data
}

template <class V, int U>
__global__ __launch_bounds__(256) void tfft_mb_write(V* __restrict__ out) {
    const size_t base = (size_t)blockIdx.x * 256 * U + threadIdx.x;
    V v;
    v.x = (float)threadIdx.x;
    v.y = 1.f;
#pragma unroll
    for (int e = 0; e < U; ++e) out[base + (size_t)e * 256] = v;
}

}  // namespace

extern "C" int turbofft_membench(int mode, const void* src_d, void* dst_d, size_t bytes, int warmup, int reps,
                                 void* stream, float* ms_per_pass) {
    if (!src_d || !dst_d || !ms_per_pass || reps < 1 || warmup < 0) { tfft_set_error("membench: bad argument"); return TURBOFFT_EINVAL; }
    const size_t tile8 = 256 * 32 * 8, tile16 = 256 * 16 * 16;     // 64 KiB per block either way
    if (bytes == 0 || bytes % tile8 || bytes / tile8 > 0x7fffffffull) { tfft_set_error("membench: bytes must be a multiple of 65536"); return TURBOFFT_EINVAL; }
    hipStream_t st = (hipStream_t)stream;
    const unsigned grid = (unsigned)(bytes / tile8);
    static_assert(tile8 == tile16, "same tile bytes for both lane widths");
    auto launch = [&]() {
        switch (mode) {
            case 0: hipLaunchKernelGGL((tfft_mb_copy<v2, 32>), dim3(grid), dim3(256), 0, st, (const v2*)src_d, (v2*)dst_d); break;
            case 1: hipLaunchKernelGGL((tfft_mb_copy<v4, 16>), dim3(grid), dim3(256), 0, st, (const v4*)src_d, (v4*)dst_d); break;
            case 2: hipLaunchKernelGGL((tfft_mb_read<v2, 32>), dim3(grid), dim3(256), 0, st, (const v2*)src_d, (float*)dst_d); break;
            default: hipLaunchKernelGGL((tfft_mb_write<v2, 32>), dim3(grid), dim3(256), 0, st, (v2*)dst_d); break;
        }
    };
    if (mode < 0 || mode > 3) { tfft_set_error("membench: mode must be 0 (copy, 8-byte lanes), 1 (copy, 16-byte lanes), 2 (read) or 3 (write)"); return TURBOFFT_EINVAL; }
    for (int i = 0; i < warmup; ++i) launch();
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess) { tfft_set_error("membench: hipEventCreate failed"); return TURBOFFT_EHIP; }
    if (hipEventCreate(&e1) != hipSuccess) { (void)hipEventDestroy(e0); tfft_set_error("membench: hipEventCreate failed"); return TURBOFFT_EHIP; }
    hipError_t e = hipEventRecord(e0, st);
    for (int i = 0; i < reps; ++i) launch();
    if (e == hipSuccess) e = hipEventRecord(e1, st);
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e == hipSuccess) e = hipGetLastError();
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (e != hipSuccess) { tfft_set_error("membench: %s", hipGetErrorString(e)); return TURBOFFT_EHIP; }
    *ms_per_pass = ms / reps;
    return TURBOFFT_OK;
}
