// Offline two-sided checksums: the baseline the fused scheme is compared with
// (include/cufft/cufft_ft.h:19-95: a checksum pass over the input, the library
// transform, a checksum pass over the output, each as its own launch).  The
// same arithmetic as the fused kernels -- re+im of sum x[m] c[m] against re+im
// of sum y[k] r[k%3], per transform -- but every pass reads its operand from
// HBM again, which is what the comparison is about.  Measurement and
// cross-check only: nothing here is used by turbofft_exec.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <vector>

#include "../../include/turbofft.h"

void tfft_set_error(const char* fmt, ...);   // turbofft_host.cpp

namespace {

template <class R> struct C2;
template <> struct C2<float> { typedef float2 T; };
template <> struct C2<double> { typedef double2 T; };

template <class R>
__device__ __forceinline__ R wsum(R v) {
    for (int d = 1; d < 64; d <<= 1) v += __shfl_xor(v, d, 64);
    return v;
}

// One wavefront per work item = CHUNK consecutive elements of one transform (a whole transform
// when N <= CHUNK); items are dealt to the wavefronts of the grid round-robin.  Lane l reads
// elements l, l+64, ... of its item -- unit stride across the wavefront -- and the wavefront's
// totals are added to the transform's two accumulators, which the caller zeroed.
// weights == nullptr: w[k] = r[k % 3] with r = (1, w3, w3^2), the output side; otherwise
// w = weights[k], the input side (c_N = W^T r).
// sums[row] += re+im of sum x*w, mags[row] += sum over lanes of |partial sum| (the fused
// kernels' magnitude, per lane of this pass instead of per thread of the FFT block).
constexpr long long CHUNK = 8192;
template <class R>
__global__ __launch_bounds__(256) void checksum_rows(const typename C2<R>::T* __restrict__ x,
                                                     const typename C2<R>::T* __restrict__ weights,
                                                     long long N, long long rows, R* __restrict__ sums, R* __restrict__ mags) {
    const long long wave = ((long long)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const long long nwaves = ((long long)gridDim.x * blockDim.x) >> 6;
    const unsigned lane = threadIdx.x & 63;
    const R s3 = (R)0.8660253882408142;
    const long long len = N < CHUNK ? N : CHUNK, per_row = N / len;
    for (long long item = wave; item < rows * per_row; item += nwaves) {
        const long long row = item / per_row, k0 = (item % per_row) * len;
        const typename C2<R>::T* p = x + row * N + k0;
        R acc = 0;
        if (weights) {
            const typename C2<R>::T* w = weights + k0;
            for (unsigned k = lane; k < (unsigned)len; k += 64) {
                const typename C2<R>::T v = p[k], c = w[k];
                acc += v.x * (c.x + c.y) + v.y * (c.x - c.y);      // re+im of v*c
            }
        } else {
            unsigned c = (unsigned)((k0 + lane) % 3);                // 64 = 1 mod 3: the class advances by one per step
            for (unsigned k = lane; k < (unsigned)len; k += 64) {
                const typename C2<R>::T v = p[k];
                const R wx = c == 0 ? (R)1 : (R)-0.5, wy = c == 0 ? (R)0 : (c == 1 ? -s3 : s3);
                acc += v.x * (wx + wy) + v.y * (wx - wy);
                c = c == 2 ? 0 : c + 1;
            }
        }
        const R tot = wsum(acc), mag = wsum(acc < 0 ? -acc : acc);
        if (lane == 0) { atomicAdd(&sums[row], tot); atomicAdd(&mags[row], mag); }
    }
}

template <class R>
__global__ void zero_rows(R* __restrict__ a, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) a[i] = 0;
}

template <class R>
__global__ void compare_rows(const R* __restrict__ in_s, const R* __restrict__ in_m, const R* __restrict__ out_s,
                             const R* __restrict__ out_m, long long rows, R smoothing, R threshold,
                             unsigned long long* __restrict__ flagged) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows) return;
    const R d = in_s[i] - out_s[i], m = in_m[i] + out_m[i];
    if ((d < 0 ? -d : d) / (smoothing + m) > threshold) atomicAdd(flagged, 1ull);
}

__global__ void zero_counter(unsigned long long* c) { *c = 0; }

struct Scratch {
    void* p = nullptr;
    ~Scratch() { if (p) (void)hipFree(p); }
};

// sums and mags are adjacent: mags == sums + rows
template <class R>
int launch_checksum(const void* x, const void* w, long long N, long long rows, R* sums, R* mags, hipStream_t st) {
    const long long per_row = N < CHUNK ? 1 : N / CHUNK, items = rows * per_row;
    const long long waves = items < 256ll * 8 * 4 ? items : 256ll * 8 * 4;      // up to 8 blocks per CU
    const int grid = (int)((waves + 3) / 4);
    hipLaunchKernelGGL((zero_rows<R>), dim3((unsigned)((2 * rows + 255) / 256)), dim3(256), 0, st, sums, 2 * rows);
    hipLaunchKernelGGL((checksum_rows<R>), dim3(grid), dim3(256), 0, st, (const typename C2<R>::T*)x,
                       (const typename C2<R>::T*)w, N, rows, sums, mags);
    return hipGetLastError() == hipSuccess ? 0 : TURBOFFT_EHIP;
}

}  // namespace

extern "C" int turbofft_offline_checksums(int logN, int datatype, const void* in_d, const void* out_d, long long bs,
                                          void* in_sums_d, void* out_sums_d, void* stream) {
    if (logN < 1 || logN > 30 || bs < 1 || !in_d || !out_d || !in_sums_d || !out_sums_d ||
        (datatype != TURBOFFT_FP32 && datatype != TURBOFFT_FP64)) {
        tfft_set_error("offline checksums: bad argument");
        return TURBOFFT_EINVAL;
    }
    const long long N = 1ll << logN;
    const size_t es = datatype == TURBOFFT_FP32 ? 8 : 16, rs = es / 2;
    std::vector<char> c((size_t)N * es);
    int rc = turbofft_build_checksum_vector(datatype, N, 0, c.data());
    if (rc) return rc;
    Scratch tab, acc;
    if (hipMalloc(&tab.p, (size_t)N * es) != hipSuccess || hipMalloc(&acc.p, (size_t)bs * rs * 4) != hipSuccess) {
        tfft_set_error("offline checksums: device allocation failed");
        return TURBOFFT_ENOMEM;
    }
    hipStream_t st = (hipStream_t)stream;
    if (hipMemcpyAsync(tab.p, c.data(), (size_t)N * es, hipMemcpyHostToDevice, st) != hipSuccess) {
        tfft_set_error("offline checksums: table upload failed");
        return TURBOFFT_EHIP;
    }
    if (datatype == TURBOFFT_FP32) {
        float* a = (float*)acc.p;
        rc = launch_checksum<float>(in_d, tab.p, N, bs, a, a + bs, st);
        if (!rc) rc = launch_checksum<float>(out_d, nullptr, N, bs, a + 2 * bs, a + 3 * bs, st);
    } else {
        double* a = (double*)acc.p;
        rc = launch_checksum<double>(in_d, tab.p, N, bs, a, a + bs, st);
        if (!rc) rc = launch_checksum<double>(out_d, nullptr, N, bs, a + 2 * bs, a + 3 * bs, st);
    }
    if (rc || hipMemcpyAsync(in_sums_d, acc.p, (size_t)bs * rs, hipMemcpyDeviceToDevice, st) != hipSuccess ||
        hipMemcpyAsync(out_sums_d, (char*)acc.p + 2 * (size_t)bs * rs, (size_t)bs * rs, hipMemcpyDeviceToDevice, st) != hipSuccess ||
        hipStreamSynchronize(st) != hipSuccess) {
        tfft_set_error("offline checksums: launch failed");
        return TURBOFFT_EHIP;
    }
    return 0;
}

extern "C" int turbofft_offline_ft_time(int logN, int datatype, const void* in_d, void* out_d, long long bs,
                                        int warmup, int reps, void* stream, float* ms_per_exec,
                                        unsigned long long* flagged_rows) {
    if (logN < 1 || logN > 30 || bs < 1 || !in_d || !out_d || !ms_per_exec || reps < 1 || warmup < 0 ||
        (datatype != TURBOFFT_FP32 && datatype != TURBOFFT_FP64)) {
        tfft_set_error("offline checksums: bad argument");
        return TURBOFFT_EINVAL;
    }
    const long long N = 1ll << logN;
    const size_t es = datatype == TURBOFFT_FP32 ? 8 : 16, rs = es / 2;
    hipStream_t st = (hipStream_t)stream;
    std::vector<char> c((size_t)N * es);
    int rc = turbofft_build_checksum_vector(datatype, N, 0, c.data());
    if (rc) return rc;
    turbofft_plan_t* plan = turbofft_plan_create(logN, datatype, 0, 0, 1, nullptr);
    if (!plan) return TURBOFFT_ENOPLAN;
    Scratch tab, sums, cnt;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    float ms = 0;
    unsigned long long flagged = 0;
    auto fail = [&](int code, const char* what) {
        tfft_set_error("offline checksums: %s", what);
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
        turbofft_plan_destroy(plan);
        return code;
    };
    if (hipMalloc(&tab.p, (size_t)N * es) != hipSuccess || hipMalloc(&sums.p, (size_t)bs * rs * 4) != hipSuccess ||
        hipMalloc(&cnt.p, sizeof(unsigned long long)) != hipSuccess)
        return fail(TURBOFFT_ENOMEM, "device allocation failed");
    if (hipMemcpy(tab.p, c.data(), (size_t)N * es, hipMemcpyHostToDevice) != hipSuccess) return fail(TURBOFFT_EHIP, "table upload failed");
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return fail(TURBOFFT_EHIP, "event creation failed");
    for (int it = 0; it < warmup + reps; ++it) {
        if (it == warmup && hipEventRecord(e0, st) != hipSuccess) return fail(TURBOFFT_EHIP, "event record failed");
        hipLaunchKernelGGL(zero_counter, dim3(1), dim3(1), 0, st, (unsigned long long*)cnt.p);
        const int grid = (int)((bs + 255) / 256);
        if (datatype == TURBOFFT_FP32) {
            float* s = (float*)sums.p;
            rc = launch_checksum<float>(in_d, tab.p, N, bs, s, s + bs, st);
            if (!rc) rc = turbofft_exec(plan, in_d, out_d, bs, stream);
            if (!rc) rc = launch_checksum<float>(out_d, nullptr, N, bs, s + 2 * bs, s + 3 * bs, st);
            if (!rc) hipLaunchKernelGGL((compare_rows<float>), dim3(grid), dim3(256), 0, st, s, s + bs, s + 2 * bs, s + 3 * bs, bs,
                                        1000.0f, 1e-3f, (unsigned long long*)cnt.p);
        } else {
            double* s = (double*)sums.p;
            rc = launch_checksum<double>(in_d, tab.p, N, bs, s, s + bs, st);
            if (!rc) rc = turbofft_exec(plan, in_d, out_d, bs, stream);
            if (!rc) rc = launch_checksum<double>(out_d, nullptr, N, bs, s + 2 * bs, s + 3 * bs, st);
            if (!rc) hipLaunchKernelGGL((compare_rows<double>), dim3(grid), dim3(256), 0, st, s, s + bs, s + 2 * bs, s + 3 * bs, bs,
                                        1000.0, 1e-3, (unsigned long long*)cnt.p);
        }
        if (rc) return fail(rc, "launch failed");
    }
    if (hipEventRecord(e1, st) != hipSuccess || hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess)
        return fail(TURBOFFT_EHIP, "timing failed");
    if (hipMemcpy(&flagged, cnt.p, sizeof flagged, hipMemcpyDeviceToHost) != hipSuccess) return fail(TURBOFFT_EHIP, "counter read failed");
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    turbofft_plan_destroy(plan);
    *ms_per_exec = ms / (float)reps;
    if (flagged_rows) *flagged_rows = flagged;
    return 0;
}
