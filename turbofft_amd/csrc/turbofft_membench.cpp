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

// AUX: cache-policy immediate of the buffer instructions (0 default, 2 non-temporal), as in the FFT kernels
typedef unsigned u2 __attribute__((ext_vector_type(2)));
typedef unsigned u4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t mb_rsrc(const void* p) { return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, -1, 0x00020000); }
template <int AUX> __device__ __forceinline__ v2 mb_ld(const v2* p, unsigned off) { const u2 t = __builtin_amdgcn_raw_buffer_load_b64(mb_rsrc(p), off, 0, AUX); v2 r; r.x = __uint_as_float(t.x); r.y = __uint_as_float(t.y); return r; }
template <int AUX> __device__ __forceinline__ v4 mb_ld(const v4* p, unsigned off) { const u4 t = __builtin_amdgcn_raw_buffer_load_b128(mb_rsrc(p), off, 0, AUX); v4 r; r.x = __uint_as_float(t.x); r.y = __uint_as_float(t.y); r.z = __uint_as_float(t.z); r.w = __uint_as_float(t.w); return r; }
template <int AUX> __device__ __forceinline__ void mb_st(v2* p, unsigned off, v2 v) { u2 t; t.x = __float_as_uint(v.x); t.y = __float_as_uint(v.y); __builtin_amdgcn_raw_buffer_store_b64(t, mb_rsrc(p), off, 0, AUX); }
template <int AUX> __device__ __forceinline__ void mb_st(v4* p, unsigned off, v4 v) { u4 t; t.x = __float_as_uint(v.x); t.y = __float_as_uint(v.y); t.z = __float_as_uint(v.z); t.w = __float_as_uint(v.w); __builtin_amdgcn_raw_buffer_store_b128(t, mb_rsrc(p), off, 0, AUX); }

// tile of this block: with `xcd_chunk` > 0 the blocks are renumbered as in the FFT kernels, so that
// each of the 8 XCDs (hardware deals block ids round-robin) works on runs of consecutive tiles
__device__ __forceinline__ size_t mb_tile(int xcd_chunk) {
    unsigned bx = blockIdx.x;
    if (xcd_chunk > 0) {
        const unsigned xc = (unsigned)xcd_chunk, span = 8u * xc, full = (gridDim.x / span) * span;
        if (bx < full) { const unsigned q = bx >> 3, xcd = bx & 7u; bx = (q / xc) * span + xcd * xc + q % xc; }
    }
    return (size_t)bx;
}

// a block of 256 threads moves one contiguous tile of 256*U vectors: every load is issued before
// the first store, as in the FFT kernels; the lanes of a wavefront touch consecutive vectors.
// Dynamic LDS that the kernels do not touch limits the blocks resident per CU, as the exchange
// buffer of an FFT kernel does.
template <class V, int U, int AUX>
__global__ __launch_bounds__(256) void tfft_mb_copy(const V* __restrict__ in, V* __restrict__ out, int xcd_chunk) {
    const size_t base = mb_tile(xcd_chunk) * 256 * U;
    const unsigned lane = threadIdx.x * (unsigned)sizeof(V);
    V r[U];
#pragma unroll
    for (int e = 0; e < U; ++e) r[e] = mb_ld<AUX>(in + base, lane + (unsigned)(e * 256 * sizeof(V)));
#pragma unroll
    for (int e = 0; e < U; ++e) mb_st<AUX>(out + base, lane + (unsigned)(e * 256 * sizeof(V)), r[e]);
}

template <class V, int U, int AUX>
__global__ __launch_bounds__(256) void tfft_mb_read(const V* __restrict__ in, float* __restrict__ sink, int xcd_chunk) {
    const size_t base = mb_tile(xcd_chunk) * 256 * U;
    const unsigned lane = threadIdx.x * (unsigned)sizeof(V);
    V r[U];
#pragma unroll
    for (int e = 0; e < U; ++e) r[e] = mb_ld<AUX>(in + base, lane + (unsigned)(e * 256 * sizeof(V)));
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < U; ++e) acc += r[e].x;
    if (acc == 123456.789f) sink[0] = acc;       // keeps the loads alive, never true for the test data
}

template <class V, int U, int AUX>
__global__ __launch_bounds__(256) void tfft_mb_write(V* __restrict__ out, int xcd_chunk) {
    const size_t base = mb_tile(xcd_chunk) * 256 * U;
    const unsigned lane = threadIdx.x * (unsigned)sizeof(V);
    V v;
    v.x = (float)threadIdx.x;
    v.y = 1.f;
#pragma unroll
    for (int e = 0; e < U; ++e) mb_st<AUX>(out + base, lane + (unsigned)(e * 256 * sizeof(V)), v);
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
    // mode: bits 0-1 the kernel (0 copy with 8-byte lanes, 1 copy with 16-byte lanes, 2 read only, 3 write only),
    // bit 2 non-temporal accesses, bit 3 XCD-aware tile order (runs of 16 tiles), bits 4-7 blocks per CU (0: no limit)
    const int kind = mode & 3, nt = (mode >> 2) & 1, xc = ((mode >> 3) & 1) ? 16 : 0, bpc = (mode >> 4) & 15;
    if (mode < 0 || mode > 255) { tfft_set_error("membench: mode is a bit field below 256 (kernel | 4 non-temporal | 8 XCD-aware order | 16 * blocks per CU)"); return TURBOFFT_EINVAL; }
    const size_t lds = bpc ? (size_t)(160 * 1024 / bpc) / 1024 * 1024 : 0;
    const void* fns[8] = {(const void*)tfft_mb_copy<v2, 32, 0>, (const void*)tfft_mb_copy<v4, 16, 0>, (const void*)tfft_mb_read<v2, 32, 0>, (const void*)tfft_mb_write<v2, 32, 0>,
                          (const void*)tfft_mb_copy<v2, 32, 2>, (const void*)tfft_mb_copy<v4, 16, 2>, (const void*)tfft_mb_read<v2, 32, 2>, (const void*)tfft_mb_write<v2, 32, 2>};
    const void* fn = fns[kind + 4 * nt];
    if (lds > 48 * 1024 && hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        tfft_set_error("membench: cannot reserve %zu bytes of LDS per block", lds);
        return TURBOFFT_EHIP;
    }
    auto launch = [&]() {
        int xca = xc;
        const void* in_a = src_d; void* out_a = dst_d;
        if (kind == 3) { void* args[2] = {&out_a, &xca}; (void)hipLaunchKernel(fn, dim3(grid), dim3(256), args, lds, st); }
        else { void* args[3] = {&in_a, &out_a, &xca}; (void)hipLaunchKernel(fn, dim3(grid), dim3(256), args, lds, st); }
    };
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
