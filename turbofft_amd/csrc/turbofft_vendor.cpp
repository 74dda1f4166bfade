// Vendor-library side-by-side: the role of profiler::cufft::test_cufft
// (include/cufft/cufft.h:14-56 fp32, :59-101 fp64) with hipFFT in the place of
// cuFFT.  hipFFT is opened at run time (dlopen), so the library itself carries
// no dependency on it; when it cannot be opened every entry point here returns
// TURBOFFT_ENOPLAN with a message and nothing else in the library is affected.
// This is measurement and cross-checking only: no transform of the library
// is ever computed by the vendor code.
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <mutex>

#include "../../include/turbofft.h"

void tfft_set_error(const char* fmt, ...);   // turbofft_host.cpp

namespace {

// the part of the hipFFT C API that is used (hipfft/hipfft.h); handles are opaque pointers
typedef void* vfft_handle;
typedef int (*fn_plan1d)(vfft_handle*, int, int, int);
typedef int (*fn_set_stream)(vfft_handle, hipStream_t);
typedef int (*fn_exec)(vfft_handle, void*, void*, int);
typedef int (*fn_destroy)(vfft_handle);
constexpr int VFFT_C2C = 0x29, VFFT_Z2Z = 0x69, VFFT_FORWARD = -1;

struct VendorLib {
    void* so = nullptr;
    fn_plan1d plan1d = nullptr;
    fn_set_stream set_stream = nullptr;
    fn_exec exec_c2c = nullptr, exec_z2z = nullptr;
    fn_destroy destroy = nullptr;
    bool tried = false;
};
VendorLib g_lib;
std::mutex g_mu;

bool load_vendor() {
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_lib.tried) return g_lib.so != nullptr;
    g_lib.tried = true;
    const char* names[] = {"libhipfft.so", "libhipfft.so.0", "/opt/rocm/lib/libhipfft.so"};
    void* so = nullptr;
    for (const char* n : names)
        if ((so = dlopen(n, RTLD_NOW | RTLD_LOCAL))) break;
    if (!so) return false;
    g_lib.plan1d = (fn_plan1d)dlsym(so, "hipfftPlan1d");
    g_lib.set_stream = (fn_set_stream)dlsym(so, "hipfftSetStream");
    g_lib.exec_c2c = (fn_exec)dlsym(so, "hipfftExecC2C");
    g_lib.exec_z2z = (fn_exec)dlsym(so, "hipfftExecZ2Z");
    g_lib.destroy = (fn_destroy)dlsym(so, "hipfftDestroy");
    if (!g_lib.plan1d || !g_lib.set_stream || !g_lib.exec_c2c || !g_lib.exec_z2z || !g_lib.destroy) {
        dlclose(so);
        return false;
    }
    g_lib.so = so;
    return true;
}

struct VendorPlan {
    vfft_handle h = nullptr;
    ~VendorPlan() { if (h) g_lib.destroy(h); }
};

int make_plan(VendorPlan& p, int logN, int datatype, long long bs, hipStream_t stream) {
    if (logN < 1 || logN > 30 || bs < 1 || bs > 0x7fffffffll || (datatype != TURBOFFT_FP32 && datatype != TURBOFFT_FP64)) {
        tfft_set_error("vendor FFT: bad shape (logN %d, bs %lld, datatype %d)", logN, bs, datatype);
        return TURBOFFT_EINVAL;
    }
    if (!load_vendor()) {
        tfft_set_error("vendor FFT: libhipfft.so could not be opened");
        return TURBOFFT_ENOPLAN;
    }
    int rc = g_lib.plan1d(&p.h, 1 << logN, datatype == TURBOFFT_FP32 ? VFFT_C2C : VFFT_Z2Z, (int)bs);
    if (rc) { p.h = nullptr; tfft_set_error("vendor FFT: hipfftPlan1d failed with %d", rc); return TURBOFFT_EHIP; }
    rc = g_lib.set_stream(p.h, stream);
    if (rc) { tfft_set_error("vendor FFT: hipfftSetStream failed with %d", rc); return TURBOFFT_EHIP; }
    return 0;
}

int run(VendorPlan& p, int datatype, const void* in_d, void* out_d) {
    int rc = (datatype == TURBOFFT_FP32 ? g_lib.exec_c2c : g_lib.exec_z2z)(p.h, const_cast<void*>(in_d), out_d, VFFT_FORWARD);
    if (rc) { tfft_set_error("vendor FFT: exec failed with %d", rc); return TURBOFFT_EHIP; }
    return 0;
}

}  // namespace

extern "C" int turbofft_vendor_available(void) {
    return load_vendor() ? 1 : 0;
}

extern "C" int turbofft_vendor_exec(int logN, int datatype, const void* in_d, void* out_d, long long bs, void* stream) {
    if (!in_d || !out_d) { tfft_set_error("vendor FFT: null buffer"); return TURBOFFT_EINVAL; }
    VendorPlan p;
    int rc = make_plan(p, logN, datatype, bs, (hipStream_t)stream);
    if (rc) return rc;
    if ((rc = run(p, datatype, in_d, out_d))) return rc;
    if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess) { tfft_set_error("vendor FFT: stream synchronisation failed"); return TURBOFFT_EHIP; }
    return 0;
}

extern "C" int turbofft_vendor_time(int logN, int datatype, const void* in_d, void* out_d, long long bs,
                                    int warmup, int reps, void* stream, float* ms_per_exec) {
    if (!in_d || !out_d || !ms_per_exec || reps < 1 || warmup < 0) { tfft_set_error("vendor FFT: bad argument"); return TURBOFFT_EINVAL; }
    hipStream_t st = (hipStream_t)stream;
    VendorPlan p;
    int rc = make_plan(p, logN, datatype, bs, st);
    if (rc) return rc;
    for (int i = 0; i < warmup; ++i)
        if ((rc = run(p, datatype, in_d, out_d))) return rc;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        if (e0) (void)hipEventDestroy(e0);
        tfft_set_error("vendor FFT: event creation failed");
        return TURBOFFT_EHIP;
    }
    float ms = 0;
    bool timed = hipEventRecord(e0, st) == hipSuccess;
    for (int i = 0; i < reps && timed && !rc; ++i) rc = run(p, datatype, in_d, out_d);     // run() sets the message
    timed = timed && !rc && hipEventRecord(e1, st) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
            hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc) return rc;
    if (!timed) { tfft_set_error("vendor FFT: event timing failed"); return TURBOFFT_EHIP; }
    *ms_per_exec = ms / (float)reps;
    return 0;
}
