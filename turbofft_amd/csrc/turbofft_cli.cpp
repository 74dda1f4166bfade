// The `turbofft` command line: same flags, modes and output lines as the
// reference driver (main.cu:75-169, include/utils/CommandLineParser.h).
//
//   --if_verify 1 --if_bench 0 --logN L --bs B   one run, compared element-wise
//        (compareData.h:4-35, tolerance 1e-4).  The reference compares with
//        cuFFT (main.cu:98-102); here the comparison values come from a plain
//        fp64 radix-2 FFT on the host that exists only for this check and is
//        never used to produce results, and then, when hipFFT can be opened,
//        from hipFFT on the same device buffers as well.
//   --if_profile 1 --if_bench 0                  timed runs for bs..bs_end step bs_gap,
//                                                hipFFT first when present (main.cu:104-110)
//   --if_bench 1                                 logN = 1..25, bs = 1..2^(28-logN)
//   --if_bench 2                                 logN = 1..25, bs = 2^(28-logN)
//   --if_bench 11/12                             the same two sweeps with hipFFT (cuFFT in the
//                                                reference, main.cu:121)
#include <hip/hip_runtime.h>
#include <dlfcn.h>

#include <algorithm>
#include <cmath>
#include <complex>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <string>
#include <vector>

#include "../../include/turbofft.h"

namespace {

struct ProgramConfig {           // CommandLineParser.h:4-25
    long long N = 0, logN = 0, bs = 0, bs_end = 0, bs_gap = 1;
    bool if_profile = false, if_verify = false;
    int if_bench = 1;
    bool if_ft = false, if_err = false;
    int datatype = 0, thread_bs = 1;
    int param_1 = 28, param_2 = 16;
    bool param_1_given = false;
    int sm_cnt = 256, smem_size = 160;
    int logN_begin = 1, logN_end = 25;
    std::string gpu = "gfx950";
    std::string param_file_path;     // empty: built-in gfx950 table
    bool param_given = false;        // --param names the CSV; otherwise --gpu selects it
    bool if_sync = false;            // also print the reference's sync-after-every-launch timing
    int ft_correction = 1;           // 1 recompute the located tile, 2 delayed batch correction
    int ft_scheme = 0;               // 0 checksums per group of tiles (the reference's current generator), 1 thread-level verification

    static void displayHelp() {
        std::cout << "Usage: program [options]\n"
                  << "Options:\n"
                  << "  --logN <value>       Set logN to <value>, which determines N as 2^<value>.\n"
                  << "  --bs <value>         Set block size to <value>.\n"
                  << "  --bs_end <value>     Set block size end to <value> (for iterative tests).\n"
                  << "  --bs_gap <value>     Set block size gap to <value> (for iterative tests).\n"
                  << "  --if_profile <0|1>   Enable (1) or disable (0) profiling.\n"
                  << "  --if_verify <0|1>    Enable (1) or disable (0) verification.\n"
                  << "  --if_bench <0|1|2|11|12> Enable (1) or disable (0) benchmarking.\n"
                  << "                           (2) for logBS + logN = 28.\n"
                  << "                           (11) for hipFFT.\n"
                  << "                           (12) for hipFFT & logBS + logN = 28.\n"
                  << "  --if_ft <0|1>        Enable (1) or disable (0) fault tolerance.\n"
                  << "  --if_err <0|1>       Enable (1) or disable (0) error injection.\n"
                  << "  --datatype <type>    0 for FP32, 1 for FP64.\n"
                  << "  --thread_bs <value>  Set batches per block to <value>.\n"
                  << "  --gpu <str>          Set GPU spec: selects param/<gpu>/param_<type>.csv (gfx950 and MI355X: the built-in table).\n"
                  << "  --param <file>       Plan CSV (overrides the one --gpu selects).\n"
                  << "  --if_sync <0|1>      Also time with a host wait after every launch, as the reference does.\n"
                  << "  --ft_correction <1|2> With --if_err: recompute the located tile (1) or delayed batch correction (2).\n"
                  << "  --ft_scheme <0|1>    With --if_ft: checksums per group of tiles (0) or thread-level verification (1).\n"
                  << "  --logN_begin/--logN_end <value>  Restrict the --if_bench sweep.\n"
                  << "  --param_1 <value>        logBS + logN of the --if_bench sweep (default 28; the reference derives it from --gpu).\n"
                  << "  -h, --help               Display this help message and exit.\n";
    }

    bool parseParameter(const char* name, const char* value) {
        if (!strcmp(name, "--logN")) { logN = atol(value); N = 1LL << atol(value); }
        else if (!strcmp(name, "--bs")) bs = atol(value);
        else if (!strcmp(name, "--bs_end")) bs_end = atol(value);
        else if (!strcmp(name, "--bs_gap")) bs_gap = atol(value);
        else if (!strcmp(name, "--if_profile")) if_profile = atol(value);
        else if (!strcmp(name, "--if_verify")) if_verify = atol(value);
        else if (!strcmp(name, "--if_ft")) if_ft = atol(value);
        else if (!strcmp(name, "--if_err")) { if_err = atol(value); if (if_err) if_ft = true; }
        else if (!strcmp(name, "--if_bench")) if_bench = atol(value);
        else if (!strcmp(name, "--datatype")) datatype = atoi(value);
        else if (!strcmp(name, "--thread_bs")) thread_bs = atoi(value);
        else if (!strcmp(name, "--gpu")) gpu = value;
        else if (!strcmp(name, "--param")) { param_file_path = value; param_given = true; }
        else if (!strcmp(name, "--if_sync")) if_sync = atol(value);
        else if (!strcmp(name, "--ft_correction")) ft_correction = atoi(value);
        else if (!strcmp(name, "--ft_scheme")) ft_scheme = atoi(value);
        else if (!strcmp(name, "--logN_begin")) logN_begin = atoi(value);
        else if (!strcmp(name, "--logN_end")) logN_end = atoi(value);
        else if (!strcmp(name, "--param_1")) { param_1 = atoi(value); param_1_given = true; }
        else return false;
        return true;
    }

    // returns 0 to continue, otherwise the exit code (+1) to leave with
    int parseCommandLine(int argc, char** argv) {
        for (int i = 1; i < argc; ++i)
            if (!strcmp(argv[i], "--help") || !strcmp(argv[i], "-h")) { displayHelp(); return EXIT_FAILURE + 1; }
        for (int i = 1; i < argc; i += 2)
            if (i + 1 >= argc || !parseParameter(argv[i], argv[i + 1])) {
                std::cerr << "Invalid or incomplete argument: " << argv[i] << std::endl;
                return EXIT_FAILURE + 1;
            }
        resolveGpu();
        return 0;
    }

    // CommandLineParser.h:93-109: --gpu picks the plan CSV (../include/param/<gpu>/param_<T>.csv
    // there) and the sweep constants (T4: logBS+logN = 26).  Here the tables live in
    // param/<gpu>/ beside the library; "gfx950" (or "MI355X") is the table compiled into it.  The
    // reference's own relative path is tried as well, so that its directory layout keeps working.
    void resolveGpu() {
        if (gpu == "T4") { if (!param_1_given) param_1 = 26; param_2 = 4; }
        if (param_given || gpu == "gfx950" || gpu == "MI355X") return;
        const std::string leaf = "/param/" + gpu + (datatype == 1 ? "/param_double2.csv" : "/param_float2.csv");
        std::vector<std::string> tries;
        Dl_info info;
        if (dladdr((const void*)&turbofft_main, &info) && info.dli_fname) {
            std::string lib = info.dli_fname;
            size_t cut = lib.find_last_of('/');
            tries.push_back((cut == std::string::npos ? std::string(".") : lib.substr(0, cut)) + leaf);
        }
        tries.push_back("../include" + leaf);
        for (const std::string& t : tries)
            if (std::ifstream(t).good()) { param_file_path = t; return; }
        param_file_path = tries.front();       // reported as "Failed to open file." when the plan is made (readCSV.h:29-31)
    }

    void displayConfig() const {      // CommandLineParser.h:112-119
        std::cout << "N: " << N << ", bs: " << bs << ", bs_end: " << bs_end << ", bs_gap: " << bs_gap << std::endl;
        std::cout << "if_profile: " << if_profile << ", if_verify: " << if_verify << ", if_bench: " << if_bench << std::endl;
        std::cout << "if_ft: " << if_ft << ", if_err: " << if_err << std::endl;
        std::cout << "datatype: " << datatype << ", thread_bs: " << thread_bs << std::endl;
        std::cout << "gpu: " << gpu << ", param_1: " << param_1 << ", param_2: " << param_2 << std::endl;
        std::cout << "sm_cnt: " << sm_cnt << "smem_size: " << smem_size << "param_file_path: "
                  << (param_file_path.empty() ? std::string("<built-in gfx950>") : param_file_path) << std::endl;
        if (if_sync || ft_correction != 1) std::cout << "if_sync: " << if_sync << ", ft_correction: " << ft_correction << std::endl;
    }
};

// host comparison values for --if_verify: iterative radix-2 DIT in fp64
void check_fft(std::vector<std::complex<double>>& a) {
    const size_t n = a.size();
    for (size_t i = 1, j = 0; i < n; ++i) {
        size_t bit = n >> 1;
        for (; j & bit; bit >>= 1) j ^= bit;
        j ^= bit;
        if (i < j) std::swap(a[i], a[j]);
    }
    for (size_t len = 2; len <= n; len <<= 1) {
        std::vector<std::complex<double>> w(len / 2);
        for (size_t k = 0; k < len / 2; ++k) {
            double ang = -2.0 * M_PI * (double)k / (double)len;
            w[k] = {cos(ang), sin(ang)};
        }
        for (size_t i = 0; i < n; i += len)
            for (size_t k = 0; k < len / 2; ++k) {
                std::complex<double> u = a[i + k], v = a[i + k + len / 2] * w[k];
                a[i + k] = u + v;
                a[i + k + len / 2] = u - v;
            }
    }
}

// compareData.h:4-35
template <class R>
void compareData(const R* res, const std::vector<std::complex<double>>& ref, long long N, double error_bound) {
    printf("Compare begin.\n");
    for (long long i = 0; i < N; ++i) {
        double rx = res[2 * i], ry = res[2 * i + 1];
        double rel = std::abs((rx - ref[i].real()) / (1 + std::abs(ref[i].real())));
        if (rel > error_bound || rx != rx) {
            printf("Error detected: res[%lld].x=%f, res_ref[%lld].x=%f, rel_error=%f\n", i, rx, i, ref[i].real(), rel);
            return;
        }
        rel = std::abs((ry - ref[i].imag()) / (1 + std::abs(ref[i].imag())));
        if (rel > error_bound || ry != ry) {
            printf("Error detected: res[%lld].y=%f, res_ref[%lld].y=%f, rel_error=%f\n", i, ry, i, ref[i].imag(), rel);
            return;
        }
    }
    printf("Compare finished.\n");
}

struct Buffers {
    void *in_d = nullptr, *out_d = nullptr;
    std::vector<char> in_h;
    size_t esize = 8;
    ~Buffers() {
        if (in_d) (void)hipFree(in_d);
        if (out_d) (void)hipFree(out_d);
    }
};

// initializeData.h:3-79: srandom(10); fp64 (random()%100-50)/1000, fp32 (random()%100-50)/100
int initializeData(Buffers& b, int datatype, long long points, bool fill) {
    b.esize = datatype == 0 ? 8 : 16;
    if (hipMalloc(&b.in_d, (size_t)points * b.esize) != hipSuccess) { printf("input allocation failed\n"); return -1; }
    if (hipMalloc(&b.out_d, (size_t)points * b.esize * 2) != hipSuccess) { printf("output allocation failed\n"); return -1; }
    srandom(10);
    long long gen = fill ? points : std::min<long long>(points, 1ll << 22);
    b.in_h.resize((size_t)gen * b.esize);
    for (long long i = 0; i < gen; ++i) {
        if (datatype == 0) {
            ((float*)b.in_h.data())[2 * i] = (float)((double)(random() % 100 - 50) / 100.0);
            ((float*)b.in_h.data())[2 * i + 1] = (float)((double)(random() % 100 - 50) / 100.0);
        } else {
            ((double*)b.in_h.data())[2 * i] = (double)(random() % 100 - 50) / 1000.0;
            ((double*)b.in_h.data())[2 * i + 1] = (double)(random() % 100 - 50) / 1000.0;
        }
    }
    // device input: the generated block repeated
    for (long long off = 0; off < points; off += gen) {
        long long cnt = std::min(gen, points - off);
        if (hipMemcpy((char*)b.in_d + (size_t)off * b.esize, b.in_h.data(), (size_t)cnt * b.esize, hipMemcpyHostToDevice) != hipSuccess)
            return -1;
    }
    return 0;
}

// test_turbofft (main.cu:4-73): warm-up, ntest timed runs, the metric line
int test_turbofft(const ProgramConfig& cfg, int logN, long long bs, int ntest, Buffers& b, std::vector<char>* result) {
    const char* csv = cfg.param_file_path.empty() ? nullptr : cfg.param_file_path.c_str();
    turbofft_plan_t* plan = turbofft_plan_create(logN, cfg.datatype, (cfg.if_ft && cfg.ft_scheme == 1) ? 2 : (int)cfg.if_ft, cfg.if_err, cfg.thread_bs, csv);
    if (!plan) { printf("turboFFT, %d: %s\n", logN, turbofft_last_error()); return -1; }
    float ms = 0;
    int rc = TURBOFFT_OK;
    if (cfg.if_err && cfg.ft_correction == 2) rc = turbofft_set_ft_params(plan, 1000.0, 1e-3, 2);
    // One warm-up execution as in the reference (main.cu:46-49), then -- for the timed sweeps --
    // as many more as fill 30 ms: the device clocks down while a plan is being made, and ten
    // timed executions of a sub-millisecond transform would otherwise be measured on the ramp.
    int warm = 1;
    if (!rc && ntest > 1) {
        float est = 0;
        rc = turbofft_time(plan, b.in_d, b.out_d, bs, 1, 2, nullptr, &est);
        if (!rc && est > 0) warm = std::max(1, std::min(2000, (int)(30.0f / est)));
    }
    if (!rc) rc = turbofft_time(plan, b.in_d, b.out_d, bs, warm, ntest, nullptr, &ms);
    if (rc) { printf("turboFFT, %d: %s\n", logN, turbofft_last_error()); turbofft_plan_destroy(plan); return rc; }
    double N = (double)(1ll << logN);
    double gflops = 5.0 * N * logN * (double)bs / ms * 1000.0 / 1e9;             // main.cu:68
    double gbs = N * (double)bs * (double)b.esize * 2.0 / ms * 1000.0 / 1e9;     // main.cu:69
    printf("turboFFT, %d, %d, %8.3f, %8.3f, %8.3f\n", logN, (int)log2((double)bs), ms, gflops, gbs);
    if (cfg.if_sync) {
        // the figure the reference's loop measures: the host waits after every launch (main.cu:53-62)
        float ms_s = 0;
        rc = turbofft_time_sync(plan, b.in_d, b.out_d, bs, 1, ntest, nullptr, &ms_s);
        if (rc) { printf("turboFFT_sync, %d: %s\n", logN, turbofft_last_error()); turbofft_plan_destroy(plan); return rc; }
        printf("turboFFT_sync, %d, %d, %8.3f, %8.3f, %8.3f\n", logN, (int)log2((double)bs), ms_s,
               5.0 * N * logN * (double)bs / ms_s * 1000.0 / 1e9, N * (double)bs * (double)b.esize * 2.0 / ms_s * 1000.0 / 1e9);
    }
    if (cfg.if_ft) {
        unsigned long long c[4] = {0, 0, 0, 0};
        turbofft_get_ft_counters(plan, &c[0], &c[1], &c[2], &c[3], nullptr, 0, nullptr);
        printf("turboFFT_ft, %d, checked=%llu, detected=%llu, corrected=%llu, uncorrectable=%llu\n", logN, c[0], c[1], c[2], c[3]);
    }
    if (result) {
        result->resize((size_t)(1ll << logN) * bs * b.esize);
        if (hipMemcpy(result->data(), b.out_d, result->size(), hipMemcpyDeviceToHost) != hipSuccess) rc = -1;   // main.cu:72
    }
    turbofft_plan_destroy(plan);
    return rc;
}

// test_cufft (cufft/cufft.h:14-56): the vendor library on the same buffers, same metric line
int test_vendor_fft(const ProgramConfig& cfg, int logN, long long bs, int ntest, Buffers& b, std::vector<char>* result) {
    float ms = 0;
    int warm = 1;
    int rc = TURBOFFT_OK;
    if (ntest > 1) {              // the same 30 ms of warm-up as for this library's plans
        float est = 0;
        rc = turbofft_vendor_time(logN, cfg.datatype, b.in_d, b.out_d, bs, 1, 2, nullptr, &est);
        if (!rc && est > 0) warm = std::max(1, std::min(2000, (int)(30.0f / est)));
    }
    if (!rc) rc = turbofft_vendor_time(logN, cfg.datatype, b.in_d, b.out_d, bs, warm, ntest, nullptr, &ms);
    if (rc) { printf("hipFFT, %d: %s\n", logN, turbofft_last_error()); return rc; }
    double N = (double)(1ll << logN);
    double gflops = 5.0 * N * logN * (double)bs / ms * 1000.0 / 1e9;             // cufft.h:41
    double gbs = N * (double)bs * (double)b.esize * 2.0 / ms * 1000.0 / 1e9;     // cufft.h:44
    printf("hipFFT, %d, %d, %8.3f, %8.3f, %8.3f\n", logN, (int)log2((double)bs), ms, gflops, gbs);
    if (result) {
        result->resize((size_t)(1ll << logN) * bs * b.esize);
        if (hipMemcpy(result->data(), b.out_d, result->size(), hipMemcpyDeviceToHost) != hipSuccess) rc = -1;   // cufft.h:46-47
    }
    return rc;
}

}  // namespace

extern "C" int turbofft_main(int argc, char** argv) {
    ProgramConfig cfg;
    int pc = cfg.parseCommandLine(argc, argv);
    if (pc) return pc - 1;
    cfg.displayConfig();
    const int ntest = 10;
    int dev_count = 0;
    if (hipGetDeviceCount(&dev_count) != hipSuccess || dev_count < 1) {
        printf("no HIP device available\n");
        return EXIT_FAILURE;
    }
    const bool vendor = turbofft_vendor_available();
    if (cfg.if_bench > 10 && !vendor) {
        printf("--if_bench %d selects hipFFT, which could not be opened (libhipfft.so).\n", cfg.if_bench);
        return EXIT_FAILURE;
    }
    if (!cfg.if_bench) {
        if (cfg.logN < 1 || cfg.bs < 1) { printf("--logN and --bs are required when --if_bench 0\n"); return EXIT_FAILURE; }
        long long bs_max = std::max(cfg.bs, cfg.bs_end);
        Buffers b;
        if (initializeData(b, cfg.datatype, cfg.N * bs_max, true)) return EXIT_FAILURE;
        if (cfg.if_verify) {
            std::vector<char> res;
            if (test_turbofft(cfg, (int)cfg.logN, cfg.bs, 1, b, &res)) return EXIT_FAILURE;
            std::vector<std::complex<double>> ref((size_t)cfg.N * cfg.bs);
            for (long long t = 0; t < cfg.bs; ++t) {
                std::vector<std::complex<double>> a((size_t)cfg.N);
                for (long long i = 0; i < cfg.N; ++i) {
                    size_t g = (size_t)(t * cfg.N + i);
                    a[i] = cfg.datatype == 0 ? std::complex<double>(((float*)b.in_h.data())[2 * g], ((float*)b.in_h.data())[2 * g + 1])
                                             : std::complex<double>(((double*)b.in_h.data())[2 * g], ((double*)b.in_h.data())[2 * g + 1]);
                }
                check_fft(a);
                std::copy(a.begin(), a.end(), ref.begin() + (size_t)t * cfg.N);
            }
            if (cfg.datatype == 0) compareData((const float*)res.data(), ref, cfg.N * cfg.bs, 1e-4);
            else compareData((const double*)res.data(), ref, cfg.N * cfg.bs, 1e-4);
            if (vendor) {                       // main.cu:99-101: the same comparison with the vendor library's result
                std::vector<char> vres;
                if (test_vendor_fft(cfg, (int)cfg.logN, cfg.bs, 1, b, &vres)) return EXIT_FAILURE;
                for (size_t i = 0; i < ref.size(); ++i)
                    ref[i] = cfg.datatype == 0 ? std::complex<double>(((float*)vres.data())[2 * i], ((float*)vres.data())[2 * i + 1])
                                               : std::complex<double>(((double*)vres.data())[2 * i], ((double*)vres.data())[2 * i + 1]);
                if (cfg.datatype == 0) compareData((const float*)res.data(), ref, cfg.N * cfg.bs, 1e-4);
                else compareData((const double*)res.data(), ref, cfg.N * cfg.bs, 1e-4);
            } else {
                printf("hipFFT could not be opened: compared with the host FFT only.\n");
            }
        }
        if (cfg.if_profile) {
            if (vendor)
                for (long long bs = cfg.bs; bs <= std::max(cfg.bs, cfg.bs_end); bs += cfg.bs_gap)
                    if (test_vendor_fft(cfg, (int)cfg.logN, bs, ntest, b, nullptr)) return EXIT_FAILURE;
            for (long long bs = cfg.bs; bs <= std::max(cfg.bs, cfg.bs_end); bs += cfg.bs_gap)
                if (test_turbofft(cfg, (int)cfg.logN, bs, ntest, b, nullptr)) return EXIT_FAILURE;
        }
        return 0;
    }
    // benchmark sweep (main.cu:114-128)
    Buffers b;
    if (initializeData(b, cfg.datatype, 1ll << cfg.param_1, false)) return EXIT_FAILURE;
    for (int logN = std::max(1, cfg.logN_begin); logN <= std::min(25, cfg.logN_end); ++logN) {
        long long bs = 1;
        if (cfg.if_bench % 10 == 2) bs <<= (cfg.param_1 - logN);
        for (int i = 0; i <= cfg.param_1 - logN; ++i) {
            if (cfg.if_bench > 10) test_vendor_fft(cfg, logN, bs, ntest, b, nullptr);
            else test_turbofft(cfg, logN, bs, ntest, b, nullptr);
            bs *= 2;
            if (cfg.if_bench % 10 == 2) break;
        }
    }
    return 0;
}
