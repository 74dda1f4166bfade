// Host driver behind the C ABI in include/turbofft.h.
//
// Mirrors the host side of the reference (main.cu:4-73 test_turbofft,
// include/utils/initializeData.h, include/utils/abft.h, include/utils/readCSV.h)
// for MI355X: plan rows come from the reference's 11-column CSV format, kernels
// from the generated registry, geometry is passed to the kernels at launch.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

#include "../../include/turbofft.h"
#include "tfft_registry.h"

extern "C" const char* tfft_builtin_param_csv(int datatype);   // generated: the gfx950 CSV text
extern "C" const char* tfft_builtin_param_ft_csv(int datatype);   // generated: rows replaced in FT plans
extern "C" const char* tfft_builtin_param_tt_csv(int datatype);   // generated: rows replaced in plans with thread-level verification
extern "C" const char* tfft_builtin_param_pair_csv(int datatype);   // generated: two-launch rows that run as one fused kernel
extern "C" const char* tfft_builtin_param_small_csv(int datatype);   // generated: rows for batches too small to fill the device

namespace {

thread_local std::string g_err;

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
    return code;
}

}  // namespace

// for the other host sources of the library (the vendor side-by-side)
void tfft_set_error(const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
}

namespace {

// A failed call is reported once, through the return code: the runtime's own record of it is
// cleared, or the caller's next check of hipGetLastError() (PyTorch makes one after every launch)
// would report this library's error as its own.
#define HIP_TRY(expr)                                                                         \
    do {                                                                                      \
        hipError_t e_ = (expr);                                                               \
        if (e_ != hipSuccess) {                                                               \
            (void)hipGetLastError();                                                          \
            return fail(TURBOFFT_EHIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), \
                        __FILE__, __LINE__);                                                  \
        }                                                                                     \
    } while (0)

constexpr double kPi = 3.14159265358979323846;
// checksum groups shared by several blocks: tiles a block walks, bytes of partial-sum slots and
// ticket words a fault-tolerant plan with longer groups holds
constexpr int kPartLen = 8;
constexpr size_t kPartSumsBytes = (size_t)128 << 20;
constexpr long long kPartTickets = 1ll << 20;
constexpr int kCuLdsBytes = 160 * 1024;     // LDS of one gfx950 compute unit
constexpr long long kFixGrid = 256;         // blocks of the launch that recomputes queued tiles
constexpr size_t kMaxSmallWs = 8;           // intermediate buffers (one per stream) a plan keeps for its small-batch row
constexpr size_t kMaxPairWs = 8;            // slot sets (one per stream) a plan keeps for its fused pair
constexpr int kPairLimitMs = 2000;          // longest wait of a block of a fused pair for other blocks
// smallest err_threshold the compact checksum tables serve: half-precision entries (fp32 kernels)
// leave up to 1e-4 of the checksum magnitude as residual on clean data, single-precision ones
// (fp64 kernels) 1e-8
constexpr double kCompactMinThreshold32 = 5e-4, kCompactMinThreshold64 = 1e-6;
constexpr double kSqrt3_2_literal = 0.8660253882408142;   // abft.h:22-28, float-rounded

struct Row {
    int v[40];           // 11 reference columns + optional per-launch flags: split exchange,
                         // prefetch, cross-lane last pass; then the tiles-per-block hint, the
                         // per-launch wavefronts-per-SIMD the plain kernel was compiled for and
                         // the per-launch non-temporal access bits, then the per-launch
                         // number of consecutive tiles an XCD works on (0 = 64), then the per-launch
                         // compact-checksum-table flag of the fault-tolerant kernel, then the per-launch
                         // number of tiles a block walks of a checksum group that several blocks share
                         // (0 = the library's default)
    // rows of fused pairs (columns 37-39): blocks per team (0: 8), transforms per piece (0: 1), teams per XCD
    // (0: as many as one block per CU gives)
    int team() const { return v[36] > 0 ? v[36] : 8; }
    int per_piece() const { return v[37] > 0 ? v[37] : 1; }
    int teams() const { return v[38]; }
    int ck(int i) const { return v[30 + i]; }
    int gp(int i) const { return v[33 + i]; }
    int nt(int i) const { return v[24 + i]; }
    int xc(int i) const { return v[27 + i]; }
    int tiles() const { return v[20]; }
    int wv(int i) const { return v[21 + i]; }
    int split(int i) const { return v[11 + i]; }
    int pf(int i) const { return v[14 + i]; }
    int xl(int i) const { return v[17 + i]; }
    int logN() const { return v[0]; }
    int launches() const { return v[1]; }
    int logNi(int i) const { return v[2 + i]; }
    int BS(int i) const { return v[5 + i]; }
    int n(int i) const { return v[8 + i]; }
};

// readCSV.h:3-33: split on ',' and atoi; row index == logN.
bool parse_csv(std::istream& in, std::vector<Row>& rows) {
    std::string line;
    while (std::getline(in, line)) {
        if (line.find_first_not_of(" \t\r\n") == std::string::npos) continue;
        if (line[line.find_first_not_of(" \t")] == '#') continue;
        Row r;
        memset(&r, 0, sizeof r);
        std::istringstream ls(line);
        std::string tok;
        int c = 0;
        while (c < 40 && std::getline(ls, tok, ',')) r.v[c++] = atoi(tok.c_str());
        if (c < 11) return false;
        rows.push_back(r);
    }
    return true;
}

int kind_of_launch(int launches, int i) {   // 0 row1, 1 col, 2 rowT
    if (launches == 1) return 0;
    return i == launches - 1 ? 2 : 1;
}

const tfft_kernel_entry* find_kernel(int datatype, int kind, int logNi, int BS, int n, int ft, int split, int pf, int xl, int wv, int nt, int inv = 0, int ck = 0) {
    int cnt = 0;
    const tfft_kernel_entry* t = tfft_kernel_table(&cnt);
    for (int i = 0; i < cnt; ++i)
        if (t[i].datatype == datatype && t[i].kind == kind && t[i].logNi == logNi && t[i].BS == BS &&
            t[i].n == n && t[i].ft == ft && t[i].split == split && t[i].pf == pf && t[i].xl == xl && t[i].wv == wv && t[i].nt == nt && t[i].inv == inv && t[i].ck == ck)
            return &t[i];
    return nullptr;
}

const tfft_pair_entry* find_pair(int datatype, const Row& r) {
    int cnt = 0;
    const tfft_pair_entry* t = tfft_pair_table(&cnt);
    for (int i = 0; i < cnt; ++i)
        if (t[i].datatype == datatype && t[i].logN1 == r.logNi(0) && t[i].BS1 == r.BS(0) && t[i].n1 == r.n(0) && t[i].split1 == (r.split(0) ? 1 : 0) &&
            t[i].nt1 == (r.nt(0) & 1) && t[i].logN2 == r.logNi(1) && t[i].BS2 == r.BS(1) && t[i].n2 == r.n(1) && t[i].split2 == (r.split(1) ? 1 : 0) &&
            t[i].nt2 == (r.nt(1) & 2))
            return &t[i];
    return nullptr;
}

template <class C>
void fill_twiddle(C* out, long long N) {
    // initializeData.h:31-37: for c = 1,2,4..N, tw[c-1+m] = exp(-2 pi i m / c)
    for (long long c = 1; c <= N; c *= 2)
        for (long long m = 0; m < c; ++m) {
            double ang = -2.0 * kPi * (double)m / (double)c;
            out[c - 1 + m].x = (decltype(out[0].x))cos(ang);
            out[c - 1 + m].y = (decltype(out[0].x))sin(ang);
        }
}

// exact c_N[i] = sum_j r[j%3] W_N^{ij}: one geometric series per residue class t = j % 3,
//   S_t = W^{it} (1 - q^{n_t}) / (1 - q),  q = W^{3i},
// with 1 - exp(-2ia) = 2i sin(a) exp(-ia) and all angles reduced in integers.
void checksum_exact(long long N, double* re, double* im) {
    const double rx[3] = {1.0, -0.5, -0.5}, ry[3] = {0.0, -kSqrt3_2_literal, kSqrt3_2_literal};
    for (long long i = 0; i < N; ++i) {
        double sx = 0, sy = 0;
        for (int t = 0; t < 3; ++t) {
            long long nt = (N - t + 2) / 3;              // # of j < N with j % 3 == t
            if (nt <= 0) continue;
            double gx, gy;                               // sum_m q^m, m < nt
            long long q3 = (3 * i) % N;
            if (q3 == 0) {
                gx = (double)nt; gy = 0;
            } else {
                double a = kPi * (double)q3 / (double)N;
                long long qb = (q3 * nt) % N;
                double b = kPi * (double)qb / (double)N;
                double mag = sin(b) / sin(a);
                double ph = -(b - a);
                gx = mag * cos(ph); gy = mag * sin(ph);
            }
            long long it = (i * t) % N;
            double wa = -2.0 * kPi * (double)it / (double)N;
            double wx = cos(wa), wy = sin(wa);
            double tx = gx * wx - gy * wy, ty = gx * wy + gy * wx;
            sx += tx * rx[t] - ty * ry[t];
            sy += tx * ry[t] + ty * rx[t];
        }
        re[i] = sx; im[i] = sy;
    }
}

// abft.h:21-61 verbatim arithmetic: angle 2*pi*i*j rounded to float before the
// division by float(N); cos/sin and the accumulation in T.
template <class C, class R>
void checksum_reference(long long N, C* dest) {
    C r[3];
    r[0].x = (R)1.0; r[0].y = (R)0.0;
    r[1].x = (R)-0.5; r[1].y = (R)-kSqrt3_2_literal;
    r[2].x = (R)-0.5; r[2].y = (R)kSqrt3_2_literal;
    for (long long i = 0; i < N; ++i) {
        dest[i].x = 0; dest[i].y = 0;
        for (long long j = 0; j < N; ++j) {
            float ang = -(float)(2 * kPi * (double)i * (double)j) / (float)N;
            R x, y;
            if (sizeof(R) == 4) { x = (R)cosf(ang); y = (R)sinf(ang); }
            else { x = (R)cos((double)ang); y = (R)sin((double)ang); }
            dest[i].x += x * r[j % 3].x - y * r[j % 3].y;
            dest[i].y += x * r[j % 3].y + y * r[j % 3].x;
        }
    }
}

struct c32 { float x, y; };
struct c64 { double x, y; };

}  // namespace

struct turbofft_plan {
    int logN = 0, datatype = 0, if_ft = 0, if_err = 0, thread_bs = 1;
    int scheme = 0;                // fault-tolerant plans: 0 block-level two-sided checksums over a group of tiles, 1 thread-level verification
    bool tiles_from_row = false;   // thread_bs is the plan row's tuned tiles-per-block, not the caller's
    Row row{};
    int launches = 0;
    const tfft_kernel_entry* k[3] = {nullptr, nullptr, nullptr};
    const tfft_kernel_entry* k_inv[3] = {nullptr, nullptr, nullptr};   // inverse plans: flavour of launch i (first and last differ from k)
    const tfft_kernel_entry* k_dc[3] = {nullptr, nullptr, nullptr};    // fault-tolerant plans: delayed-batch-correction flavour of launch i (may be absent)
    const tfft_kernel_entry* k_full[3] = {nullptr, nullptr, nullptr};  // where k[i] reads the compact checksum table: the flavour with the full table
    void* cksum16[3] = {nullptr, nullptr, nullptr};                    // compact checksum tables (half-precision cotangents), launches whose k[i] reads one
    int tb_gap[3] = {1, 1, 1};
    int resident[3] = {1, 1, 1};   // blocks of launch i that fit on the device at once
    size_t esize = 8;
    // device tables
    void* tw = nullptr;          // concatenated twiddle table, 2*tw_N - 1 entries
    long long tw_N = 0;
    void* tw_lo[3] = {nullptr, nullptr, nullptr};
    int lo_bits[3] = {0, 0, 0};
    void* cksum[3] = {nullptr, nullptr, nullptr};
    unsigned long long* counters = nullptr;   // 8 x u64
    long long* flagged = nullptr;
    int flagged_cap = 4096;
    // Checksum groups shared by several blocks (plans whose groups are longer than ft_part_len
    // tiles): slots for the blocks' partial checksums and one ticket word per group, sized once
    // at plan creation; an execution that would need more walks whole groups per block.
    int ft_part_len[3] = {0, 0, 0};           // tiles per block (0: the whole group)
    void* part_sums = nullptr;
    unsigned* tickets = nullptr;
    long long* fix_list = nullptr;            // tiles_n slots: tiles the fix-up launch recomputes
    unsigned* fix_ctl = nullptr;              // queue length, finished blocks of the fix-up launch
    size_t part_sums_bytes = 0;
    long long tickets_n = 0;
    // FT run-time parameters
    double err_smoothing = 1000.0, err_threshold = 1e-3;
    int correct = 0;
    int inj_mode = 0, inj_launch = -1, inj_every = 1, inj_s = 0, inj_m = 0;
    long long inj_tile = 0;
    double inj_mag = 100.0;
    int cksum_mode = 0;
    int xcd_chunk = -1;          // TURBOFFT_XCD_CHUNK: tiles per XCD chunk for every launch (0 = plain block order); -1 = unset
    int xcd_chunk_l[3] = {64, 64, 64};   // per launch: the plan row's value, else 64
    // stream of the most recent execution: the counter queries wait for it, not for the device
    std::atomic<void*> last_stream{nullptr};
    // Small batches (plain built-in plans): a second row of narrow tiles in two launches that
    // spreads few transforms over many CUs.  `small` is a plan of its own for that row; it runs
    // for bs <= small_max_bs.  Its intermediate lives in the upper half of the caller's `out`
    // when this plan is a multi-launch one too, else in a buffer of `small_ws` (N * small_max_bs
    // elements each).
    turbofft_plan* small = nullptr;
    long long small_max_bs = 0;
    // one intermediate buffer per stream that has run a small batch (single-launch main rows only):
    // executions on different streams never share one; the first is allocated with the plan
    struct SmallWs { void* stream; bool assigned; void* buf; };
    std::vector<SmallWs> small_ws;
    std::mutex small_mu;
    bool small_enabled = true;
    // Fused pair (plain built-in two-launch plans): a row whose two launches run as ONE kernel, the
    // intermediate staying in slots that the XCDs' L2s hold.  `pair` is a plan of its own for that row
    // (tables, launch geometry); the fields below it are set on that plan.  Every stream that has run
    // the pair owns a set of slots and a control block, so executions on different streams share none.
    turbofft_plan* pair = nullptr;
    const tfft_pair_entry* pk = nullptr;
    int pair_team = 0, pair_per_piece = 0, pair_grid = 0, pair_teams_per_xcd = 0, pair_limit_ms = kPairLimitMs;
    struct PairWs { void* stream; bool assigned; void* slots; unsigned* ctl; unsigned* err_host; unsigned long long* prof; };
    bool pair_prof = false;           // TURBOFFT_FUSED_PROF=1 at plan creation: diagnostic builds of the kernel leave their timings per execution
    std::vector<PairWs> pair_ws;
    std::mutex pair_mu;
    bool pair_enabled = true;
    bool compact_enabled = true;      // TURBOFFT_COMPACT_CHECKSUM=0 keeps the full-table kernels
};

extern "C" {

const char* turbofft_last_error(void) { return g_err.c_str(); }

int turbofft_build_twiddle_table(int datatype, long long N, void* out) {
    if (!out) return fail(TURBOFFT_EINVAL, "twiddle table: null output buffer");
    if (N < 1 || (N & (N - 1))) return fail(TURBOFFT_EINVAL, "twiddle table: N must be a power of two");
    if (datatype == TURBOFFT_FP32) fill_twiddle((c32*)out, N);
    else if (datatype == TURBOFFT_FP64) fill_twiddle((c64*)out, N);
    else return fail(TURBOFFT_EINVAL, "bad datatype %d", datatype);
    return TURBOFFT_OK;
}

int turbofft_build_checksum_vector(int datatype, long long N, int mode, void* out) {
    if (!out) return fail(TURBOFFT_EINVAL, "checksum vector: null output buffer");
    if (N < 2 || (N & (N - 1))) return fail(TURBOFFT_EINVAL, "checksum vector: N must be a power of two >= 2");
    if (datatype != TURBOFFT_FP32 && datatype != TURBOFFT_FP64) return fail(TURBOFFT_EINVAL, "bad datatype %d", datatype);
    if (mode == 1) {
        if (datatype == TURBOFFT_FP32) checksum_reference<c32, float>(N, (c32*)out);
        else checksum_reference<c64, double>(N, (c64*)out);
        return TURBOFFT_OK;
    }
    if (mode != 0) return fail(TURBOFFT_EINVAL, "checksum mode must be 0 (exact) or 1 (reference)");
    std::vector<double> re(N), im(N);
    checksum_exact(N, re.data(), im.data());
    for (long long i = 0; i < N; ++i) {
        if (datatype == TURBOFFT_FP32) { ((c32*)out)[i].x = (float)re[i]; ((c32*)out)[i].y = (float)im[i]; }
        else { ((c64*)out)[i].x = re[i]; ((c64*)out)[i].y = im[i]; }
    }
    return TURBOFFT_OK;
}

int turbofft_builtin_plan_row(int datatype, int logN, int row[11]) {
    if (datatype != TURBOFFT_FP32 && datatype != TURBOFFT_FP64) return fail(TURBOFFT_EINVAL, "bad datatype %d", datatype);
    std::istringstream in(tfft_builtin_param_csv(datatype));
    std::vector<Row> rows;
    if (!parse_csv(in, rows)) return fail(TURBOFFT_ENOPLAN, "built-in plan table is malformed");
    if (logN < 0 || logN >= (int)rows.size() || rows[logN].launches() == 0)
        return fail(TURBOFFT_ENOPLAN, "no built-in plan row for logN=%d", logN);
    memcpy(row, rows[logN].v, sizeof(int) * 11);
    return TURBOFFT_OK;
}

int turbofft_kernel_count(void) {
    int c = 0;
    tfft_kernel_table(&c);
    return c;
}

const char* turbofft_kernel_name(int i) {
    int c = 0;
    const tfft_kernel_entry* t = tfft_kernel_table(&c);
    return (i >= 0 && i < c) ? t[i].name : nullptr;
}

void turbofft_plan_destroy(turbofft_plan_t* p) {
    if (!p) return;
    if (p->small) turbofft_plan_destroy(p->small);
    if (p->pair) turbofft_plan_destroy(p->pair);
    for (auto& w : p->pair_ws) {
        if (w.slots) (void)hipFree(w.slots);
        if (w.ctl) (void)hipFree(w.ctl);
        if (w.err_host) (void)hipHostFree(w.err_host);
        if (w.prof) (void)hipFree(w.prof);
    }
    for (auto& w : p->small_ws) if (w.buf) (void)hipFree(w.buf);
    if (p->tw) (void)hipFree(p->tw);
    for (int i = 0; i < 3; ++i) {
        if (p->tw_lo[i]) (void)hipFree(p->tw_lo[i]);
        if (p->cksum[i]) (void)hipFree(p->cksum[i]);
        if (p->cksum16[i]) (void)hipFree(p->cksum16[i]);
    }
    if (p->counters) (void)hipFree(p->counters);
    if (p->flagged) (void)hipFree(p->flagged);
    if (p->part_sums) (void)hipFree(p->part_sums);
    if (p->tickets) (void)hipFree(p->tickets);
    if (p->fix_list) (void)hipFree(p->fix_list);
    if (p->fix_ctl) (void)hipFree(p->fix_ctl);
    delete p;
}

// (re)build the per-launch checksum tables in the plan's current mode and copy them to the device
static int upload_checksum_tables(turbofft_plan* p) {
    for (int i = 0; i < p->launches; ++i) {
        long long Ni = 1ll << p->row.logNi(i);
        std::vector<char> host((size_t)Ni * p->esize);
        int rc = turbofft_build_checksum_vector(p->datatype, Ni, p->cksum_mode, host.data());
        if (rc) return rc;
        // device form: (re c + im c, re c - im c)
        for (long long m = 0; m < Ni; ++m) {
            if (p->datatype == TURBOFFT_FP32) { c32& v = ((c32*)host.data())[m]; float a = v.x + v.y, b = v.x - v.y; v.x = a; v.y = b; }
            else { c64& v = ((c64*)host.data())[m]; double a = v.x + v.y, b = v.x - v.y; v.x = a; v.y = b; }
        }
        HIP_TRY(hipMemcpy(p->cksum[i], host.data(), host.size(), hipMemcpyHostToDevice));
        if (p->k[i] && p->k[i]->ck) {
            // compact form (exact angles only): t[m] = cot(pi (m/Ni + 1/3)) in half precision, two
            // elements of a thread per word: word [x + Tr*q] = (t[x + Tr*2q], t[x + Tr*(2q+1)])
            const long long Tr = Ni / p->row.n(i);
            auto cot = [&](long long m) { const double a = kPi * (double)(3 * m + Ni) / (double)(3 * Ni); return cos(a) / sin(a); };
            std::vector<unsigned> words;
            if (p->datatype == TURBOFFT_FP32) {
                auto half_bits = [&](long long m) -> unsigned {
                    const _Float16 h = (_Float16)(float)cot(m);
                    unsigned short b;
                    memcpy(&b, &h, sizeof b);
                    return b;
                };
                words.resize((size_t)(Ni / 2));
                for (long long q = 0; q < p->row.n(i) / 2; ++q)
                    for (long long x = 0; x < Tr; ++x)
                        words[(size_t)(x + Tr * q)] = half_bits(x + Tr * 2 * q) | (half_bits(x + Tr * (2 * q + 1)) << 16);
            } else {
                // fp64 kernels: single precision, one word per element, natural order
                words.resize((size_t)Ni);
                for (long long m = 0; m < Ni; ++m) {
                    const float f = (float)cot(m);
                    memcpy(&words[(size_t)m], &f, sizeof f);
                }
            }
            if (!p->cksum16[i]) HIP_TRY(hipMalloc(&p->cksum16[i], words.size() * sizeof(unsigned)));
            HIP_TRY(hipMemcpy(p->cksum16[i], words.data(), words.size() * sizeof(unsigned), hipMemcpyHostToDevice));
        }
    }
    return TURBOFFT_OK;
}

namespace { int static_workspace(void** ptr); }

static int plan_build_row(turbofft_plan* p, const Row& row);

// One more set of slots and a control block for the fused pair of plan `p` (`q` is the pair's own plan).
// False when the memory cannot be had; nothing is kept then.
static bool pair_add_ws(turbofft_plan* p, const turbofft_plan* q, void* stream, bool assigned) {
    const size_t nslots = (size_t)8 * q->pair_teams_per_xcd;
    const size_t slot_bytes = ((size_t)q->pair_per_piece << q->logN) * q->esize;
    const size_t ctl_bytes = sizeof(unsigned) * TFFT_FUSE_CTL_WORDS(nslots);
    void *sl = nullptr, *ctl = nullptr, *eh = nullptr, *pf = nullptr;
    const size_t prof_bytes = (size_t)8 * sizeof(unsigned long long) * (size_t)q->pair_grid;
    bool ok = hipMalloc(&sl, nslots * slot_bytes) == hipSuccess && hipMalloc(&ctl, ctl_bytes) == hipSuccess &&
              hipHostMalloc(&eh, 64, hipHostMallocDefault) == hipSuccess && hipMemset(ctl, 0, ctl_bytes) == hipSuccess &&
              (!q->pair_prof || (hipMalloc(&pf, prof_bytes) == hipSuccess && hipMemset(pf, 0, prof_bytes) == hipSuccess));
    if (!ok) {
        (void)hipGetLastError();
        if (sl) (void)hipFree(sl);
        if (ctl) (void)hipFree(ctl);
        if (eh) (void)hipHostFree(eh);
        if (pf) (void)hipFree(pf);
        return false;
    }
    *(volatile unsigned*)eh = 0u;
    p->pair_ws.push_back({stream, assigned, sl, (unsigned*)ctl, (unsigned*)eh, (unsigned long long*)pf});
    return true;
}

static int plan_build(turbofft_plan* p, const char* param_csv) {
    std::vector<Row> rows;
    if (param_csv) {
        std::ifstream f(param_csv);
        if (!f.is_open()) return fail(TURBOFFT_ENOPLAN, "Failed to open file. (%s)", param_csv);   // readCSV.h:29-31
        if (!parse_csv(f, rows)) return fail(TURBOFFT_ENOPLAN, "malformed plan CSV %s", param_csv);
    } else {
        std::istringstream in(tfft_builtin_param_csv(p->datatype));
        if (!parse_csv(in, rows)) return fail(TURBOFFT_ENOPLAN, "built-in plan table is malformed");
        if (p->if_ft && p->scheme == 0) {
            // the checksum flavour of a kernel needs more registers: where another tile shape
            // measured faster with checksums, the built-in table carries a replacement row
            std::istringstream fin(tfft_builtin_param_ft_csv(p->datatype));
            std::vector<Row> repl;
            if (!parse_csv(fin, repl)) return fail(TURBOFFT_ENOPLAN, "built-in fault-tolerant plan table is malformed");
            for (const Row& r : repl)
                if (r.logN() >= 0 && r.logN() < (int)rows.size()) rows[r.logN()] = r;
        } else if (p->if_ft) {
            // thread-level verification runs the plain rows, except where its two sums beside the data cost a
            // wavefront per SIMD and another shape measured faster
            std::istringstream fin(tfft_builtin_param_tt_csv(p->datatype));
            std::vector<Row> repl;
            if (!parse_csv(fin, repl)) return fail(TURBOFFT_ENOPLAN, "built-in thread-level plan table is malformed");
            for (const Row& r : repl)
                if (r.logN() >= 0 && r.logN() < (int)rows.size()) rows[r.logN()] = r;
        }
    }
    if (p->logN < 1 || p->logN >= (int)rows.size() || rows[p->logN].launches() < 1 || rows[p->logN].launches() > 3)
        return fail(TURBOFFT_ENOPLAN, "no plan row for logN=%d", p->logN);
    int rc = plan_build_row(p, rows[p->logN]);
    if (rc) return rc;
    if (!param_csv && !p->if_ft) {
        // the row of narrow tiles for batches that leave most of the device idle, if the
        // built-in table has one for this size (its column 21 is the largest batch it serves)
        std::istringstream sin(tfft_builtin_param_small_csv(p->datatype));
        std::vector<Row> small;
        if (!parse_csv(sin, small)) return fail(TURBOFFT_ENOPLAN, "built-in small-batch plan table is malformed");
        for (const Row& sr : small) {
            if (sr.logN() != p->logN || sr.launches() < 2 || sr.tiles() < 1) continue;
            turbofft_plan* q = new turbofft_plan();
            q->logN = p->logN; q->datatype = p->datatype; q->thread_bs = 1; q->xcd_chunk = p->xcd_chunk;
            Row clean = sr;
            clean.v[20] = 0;                      // column 21 is the batch cap here, not tiles per block
            rc = plan_build_row(q, clean);
            if (rc) { turbofft_plan_destroy(q); return rc; }
            p->small = q;
            p->small_max_bs = sr.tiles();
            if (p->launches == 1) {
                void* buf = nullptr;
                HIP_TRY(hipMalloc(&buf, ((size_t)p->small_max_bs << p->logN) * p->esize));
                p->small_ws.push_back({nullptr, false, buf});
            }
            break;
        }
    }
    // (measured at parity with the two launches at best, so a plan holds it only when asked to: TURBOFFT_FUSED=1)
    const char* fenv = getenv("TURBOFFT_FUSED");
    if (!param_csv && !p->if_ft && fenv && atoi(fenv) == 1) {
        // the row whose two launches run as one kernel, if the built-in table has one for this size
        std::vector<Row> pairs;
        if (const char* pcsv = getenv("TURBOFFT_FUSED_CSV")) {
            // tuning aid: another table of fused rows (its kernels must have been built: build.py --extra <type>:<csv>:pair)
            std::ifstream pf(pcsv);
            if (!pf.is_open() || !parse_csv(pf, pairs)) return fail(TURBOFFT_ENOPLAN, "cannot read the fused-pair table %s", pcsv);
        } else {
            std::istringstream pin(tfft_builtin_param_pair_csv(p->datatype));
            if (!parse_csv(pin, pairs)) return fail(TURBOFFT_ENOPLAN, "built-in fused-pair plan table is malformed");
        }
        for (const Row& pr : pairs) {
            if (pr.logN() != p->logN || pr.launches() != 2) continue;
            const tfft_pair_entry* pk = find_pair(p->datatype, pr);
            if (!pk) return fail(TURBOFFT_ENOPLAN, "no compiled fused pair for logN=%d", p->logN);
            turbofft_plan* q = new turbofft_plan();
            q->logN = p->logN; q->datatype = p->datatype; q->thread_bs = 1; q->xcd_chunk = p->xcd_chunk;
            Row clean = pr;
            clean.v[20] = 0;
            rc = plan_build_row(q, clean);
            if (rc) { turbofft_plan_destroy(q); return rc; }
            int dev = 0, occ = 0;
            hipDeviceProp_t prop;
            if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) { (void)hipGetLastError(); turbofft_plan_destroy(q); return fail(TURBOFFT_EHIP, "cannot query the device"); }
            if (pk->lds_bytes > kCuLdsBytes) { turbofft_plan_destroy(q); return fail(TURBOFFT_ENOPLAN, "fused pair %s needs %d B of LDS", pk->name, pk->lds_bytes); }
            if ((size_t)pk->lds_bytes > (size_t)prop.sharedMemPerBlock &&
                hipFuncSetAttribute(pk->func, hipFuncAttributeMaxDynamicSharedMemorySize, pk->lds_bytes) != hipSuccess) {
                (void)hipGetLastError(); turbofft_plan_destroy(q); return fail(TURBOFFT_EHIP, "cannot opt %s into %d B of LDS", pk->name, pk->lds_bytes);
            }
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, pk->func, pk->threads, pk->lds_bytes) != hipSuccess || occ < 1) {
                (void)hipGetLastError(); turbofft_plan_destroy(q); return fail(TURBOFFT_ENOPLAN, "fused pair %s does not fit on a CU", pk->name);
            }
            // every block of the grid has to be resident at once (blocks wait for their team): the row's number of
            // teams on each of the 8 XCDs, at most what fits there
            q->pk = pk;
            q->pair_team = pr.team();
            q->pair_per_piece = pr.per_piece();
            const int cus_per_xcd = prop.multiProcessorCount / 8, fit = cus_per_xcd * occ / q->pair_team;
            q->pair_teams_per_xcd = pr.teams() > 0 ? (pr.teams() < fit ? pr.teams() : fit) : cus_per_xcd / q->pair_team;
            q->pair_grid = 8 * q->pair_teams_per_xcd * q->pair_team;
            // (a negative limit makes every block give up at once and leave: how the tests reach the error path)
            if (const char* e = getenv("TURBOFFT_FUSED_LIMIT_MS")) if (atoi(e) != 0) q->pair_limit_ms = atoi(e);
            if (const char* e = getenv("TURBOFFT_FUSED_PROF")) q->pair_prof = atoi(e) != 0;
            if (q->pair_teams_per_xcd < 1 || q->pair_teams_per_xcd > 64) { turbofft_plan_destroy(q); break; }   // no room for a team: the plan keeps its two launches
            p->pair = q;
            if (!pair_add_ws(p, q, nullptr, false)) { turbofft_plan_destroy(q); p->pair = nullptr; return fail(TURBOFFT_ENOMEM, "no memory for the slots of the fused pair"); }
            break;
        }
    }
    return TURBOFFT_OK;
}

// A kernel whose dynamic LDS exceeds the default per-block limit has to be opted in; one that
// exceeds what a CU holds is refused here, before the runtime is asked.
static int allow_lds(const tfft_kernel_entry* k, const hipDeviceProp_t& prop) {
    if (k->lds_bytes > kCuLdsBytes)
        return fail(TURBOFFT_ENOPLAN, "kernel %s needs %d B of LDS, a gfx950 CU has %d", k->name, k->lds_bytes, kCuLdsBytes);
    if ((size_t)k->lds_bytes > (size_t)prop.sharedMemPerBlock)
        HIP_TRY(hipFuncSetAttribute(k->func, hipFuncAttributeMaxDynamicSharedMemorySize, k->lds_bytes));
    return TURBOFFT_OK;
}

static int plan_build_row(turbofft_plan* p, const Row& row) {
    p->row = row;
    const Row& r = p->row;
    if (r.logN() != p->logN) return fail(TURBOFFT_ENOPLAN, "plan row %d describes logN=%d", p->logN, r.logN());
    p->launches = r.launches();
    // Without checksums the number of tiles a block walks is a pure tuning knob: a caller that
    // leaves thread_bs at its default gets the value tuned for this size (large tiles amortise
    // the block launch over several of them).  With fault tolerance thread_bs is the checksum
    // group size and stays what the caller asked for.
    if (!p->if_ft && p->thread_bs == 1 && r.tiles() > 1) { p->thread_bs = r.tiles(); p->tiles_from_row = true; }
    int sum = 0;
    for (int i = 0; i < p->launches; ++i) sum += r.logNi(i);
    if (sum != p->logN) return fail(TURBOFFT_ENOPLAN, "plan row for logN=%d: digit sizes sum to %d", p->logN, sum);
    p->esize = p->datatype == TURBOFFT_FP32 ? 8 : 16;

    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, dev));

    long long twN = 1;
    for (int i = 0; i < p->launches; ++i) {
        int kind = kind_of_launch(p->launches, i);
        const tfft_kernel_entry* k = p->scheme == 1
            // thread-level verification runs the plain rows: same shape, exchange form and cache policy, no register budget hint
            ? find_kernel(p->datatype, kind, r.logNi(i), r.BS(i), r.n(i), 3, r.split(i) ? 1 : 0, 0, 0, 0, r.nt(i) & 3)
            : find_kernel(p->datatype, kind, r.logNi(i), r.BS(i), r.n(i), p->if_ft, r.split(i) ? 1 : 0, (p->if_ft && r.pf(i) > 1) ? 0 : r.pf(i),
                                                 (r.xl(i) && !p->if_ft) ? 1 : 0,    // FT plans keep the LDS path
                                                 p->if_ft ? 0 : r.wv(i), p->if_ft ? (r.nt(i) & 3) : r.nt(i));   // wave budget and priority bit: plain kernels only
        if (!k)
            return fail(TURBOFFT_ENOPLAN, "no compiled kernel for launch %d of logN=%d (type %d kind %d logNi %d BS %d n %d ft %d split %d prefetch %d)",
                        i, p->logN, p->datatype, kind, r.logNi(i), r.BS(i), r.n(i), p->if_ft, r.split(i), r.pf(i));
        p->k_full[i] = k;
        if (p->if_ft && p->scheme == 0 && r.ck(i)) {
            // the row asks for the flavour that reads the compact checksum table; the full-table
            // flavour stays available for the table modes and thresholds the compact form cannot serve
            const tfft_kernel_entry* kc = find_kernel(p->datatype, kind, r.logNi(i), r.BS(i), r.n(i), 1, r.split(i) ? 1 : 0, 0, 0, r.wv(i), r.nt(i) & 3, 0, r.ck(i));
            if (!kc) return fail(TURBOFFT_ENOPLAN, "no compiled compact-checksum kernel for launch %d of logN=%d", i, p->logN);
            // the largest cotangent is about 3*Ni/pi: beyond 2^16 points it leaves the half-precision range
            if (p->datatype == TURBOFFT_FP32 && r.logNi(i) > 16)
                return fail(TURBOFFT_ENOPLAN, "launch %d of logN=%d: the half-precision compact checksum table serves sub-FFTs of up to 2^16 points", i, p->logN);
            if (int rc = allow_lds(kc, prop)) return rc;
            k = kc;
        }
        p->k[i] = k;
        if (p->if_ft && p->scheme == 0) {
            p->k_dc[i] = find_kernel(p->datatype, kind, r.logNi(i), r.BS(i), r.n(i), 2, r.split(i) ? 1 : 0, 0, 0, 0, r.nt(i) & 3);
            if (p->k_dc[i] && p->k_dc[i]->lds_bytes > kCuLdsBytes) p->k_dc[i] = nullptr;   // no such flavour on this device
            if (p->k_dc[i]) if (int rc = allow_lds(p->k_dc[i], prop)) return rc;
        }
        if (r.xc(i) > 0) p->xcd_chunk_l[i] = r.xc(i);
        // Inverse plans run the same launches with a component-swapping flavour of the first and
        // the last one (plain plans only; absent for a caller's CSV whose kernels were built
        // without them, and then turbofft_exec_inverse reports it).
        p->k_inv[i] = k;
        if (!p->if_ft && (i == 0 || i == p->launches - 1)) {
            p->k_inv[i] = find_kernel(p->datatype, kind, r.logNi(i), r.BS(i), r.n(i), 0, r.split(i) ? 1 : 0, r.pf(i) > 1 ? 0 : r.pf(i),
                                      r.xl(i) ? 1 : 0, r.wv(i), r.nt(i), 1);
            if (p->k_inv[i]) if (int rc = allow_lds(p->k_inv[i], prop)) return rc;
        } else if (p->if_ft) {
            p->k_inv[i] = nullptr;
        }
        if (int rc = allow_lds(k, prop)) return rc;
        if (p->k_full[i] != k) if (int rc = allow_lds(p->k_full[i], prop)) return rc;
        int nb = 0;
        HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, k->func, k->threads, k->lds_bytes));
        if (nb < 1) return fail(TURBOFFT_ENOPLAN, "kernel %s does not fit on a CU (LDS %d B)", k->name, k->lds_bytes);
        p->tb_gap[i] = nb * prop.multiProcessorCount;      // fft_codegen.py:216-218 with measured residency
        p->resident[i] = p->tb_gap[i];
        if ((1ll << r.logNi(i)) > twN) twN = 1ll << r.logNi(i);
        if (kind == 1) {
            // inter-launch twiddle W_(2^L)^e, L = log2(Ni * ncols): e = hi << lo_bits | lo
            int L = 0;
            for (int j = i; j < p->launches; ++j) L += r.logNi(j);
            p->lo_bits[i] = (L + 1) / 2;
            long long hiN = 1ll << (L - p->lo_bits[i]);
            if (hiN > twN) twN = hiN;
            if ((1 << r.logNi(i)) * (long long)r.BS(i) < 1) return fail(TURBOFFT_EINVAL, "bad tile");
        }
    }
    // tile shape constraints
    for (int i = 0; i < p->launches; ++i) {
        int kind = kind_of_launch(p->launches, i);
        if (kind == 1) {
            int log_ncols = 0;
            for (int j = i + 1; j < p->launches; ++j) log_ncols += r.logNi(j);
            if (r.BS(i) > (1 << log_ncols)) return fail(TURBOFFT_ENOPLAN, "launch %d: BS %d exceeds %d columns", i, r.BS(i), 1 << log_ncols);
        } else if (kind == 2) {
            if (r.BS(i) > (1 << r.logNi(0))) return fail(TURBOFFT_ENOPLAN, "launch %d: BS %d exceeds the %d rows of the outer digit", i, r.BS(i), 1 << r.logNi(0));
        }
    }
    p->tw_N = twN;
    {
        std::vector<char> host((size_t)(2 * twN) * p->esize);
        turbofft_build_twiddle_table(p->datatype, twN, host.data());
        HIP_TRY(hipMalloc(&p->tw, host.size()));
        HIP_TRY(hipMemcpy(p->tw, host.data(), (size_t)(2 * twN - 1) * p->esize, hipMemcpyHostToDevice));
    }
    for (int i = 0; i < p->launches; ++i) {
        if (kind_of_launch(p->launches, i) == 1) {
            int L = 0;
            for (int j = i; j < p->launches; ++j) L += r.logNi(j);
            long long cnt = 1ll << p->lo_bits[i];
            std::vector<char> host((size_t)cnt * p->esize);
            for (long long l = 0; l < cnt; ++l) {
                double ang = -2.0 * kPi * (double)l / (double)(1ll << L);
                if (p->datatype == TURBOFFT_FP32) { ((c32*)host.data())[l].x = (float)cos(ang); ((c32*)host.data())[l].y = (float)sin(ang); }
                else { ((c64*)host.data())[l].x = cos(ang); ((c64*)host.data())[l].y = sin(ang); }
            }
            HIP_TRY(hipMalloc(&p->tw_lo[i], host.size()));
            HIP_TRY(hipMemcpy(p->tw_lo[i], host.data(), host.size(), hipMemcpyHostToDevice));
        }
    }
    if (p->if_ft && p->scheme == 0) {
        for (int i = 0; i < p->launches; ++i)
            HIP_TRY(hipMalloc(&p->cksum[i], ((size_t)1 << r.logNi(i)) * p->esize));
        int rc = upload_checksum_tables(p);
        if (rc) return rc;
    }
    if (p->launches > 1) {
        // look the static workspace of this device up now, so that turbofft_exec_static finds it
        // ready (a failure is reported by that call, which tries again)
        void* ws = nullptr;
        if (static_workspace(&ws) != TURBOFFT_OK) g_err.clear();
    }
    if (p->if_ft) {
        HIP_TRY(hipMalloc((void**)&p->counters, TFFT_FT_COUNTER_WORDS * sizeof(unsigned long long)));
        HIP_TRY(hipMemset(p->counters, 0, TFFT_FT_COUNTER_WORDS * sizeof(unsigned long long)));
        HIP_TRY(hipMalloc((void**)&p->flagged, sizeof(long long) * 2 * p->flagged_cap));
        HIP_TRY(hipMemset(p->flagged, 0xff, sizeof(long long) * 2 * p->flagged_cap));
        // Long groups are walked by several blocks, kPartLen tiles each (TURBOFFT_FT_PART_LEN
        // overrides, 0 switches it off): a block that walks many tiles in sequence gives up the
        // overlap that block scheduling provides, and few long groups leave CUs idle.
        int part_len = kPartLen;
        if (const char* e = getenv("TURBOFFT_FT_PART_LEN")) part_len = atoi(e);
        if (part_len > 0 && p->thread_bs > part_len && p->scheme == 0) {
            // (a plan row may name its own length per launch, columns 34-36 of the fault-tolerant table; groups of up to
            // kPartLen tiles are never shared, whatever the row says: sharing them measured slower at most sizes)
            for (int i = 0; i < p->launches; ++i) p->ft_part_len[i] = (p->row.gp(i) > 0 && !getenv("TURBOFFT_FT_PART_LEN")) ? p->row.gp(i) : part_len;
            // (the slots themselves are allocated by the first execution that shares a group)
        }
    }
    return TURBOFFT_OK;
}

turbofft_plan_t* turbofft_plan_create(int logN, int datatype, int if_ft, int if_err, int thread_bs,
                                      const char* param_csv) {
    g_err.clear();
    if (datatype != TURBOFFT_FP32 && datatype != TURBOFFT_FP64) { fail(TURBOFFT_EINVAL, "bad datatype %d", datatype); return nullptr; }
    if (thread_bs < 1) { fail(TURBOFFT_EINVAL, "thread_bs must be >= 1"); return nullptr; }
    if (if_ft < 0 || if_ft > 2) { fail(TURBOFFT_EINVAL, "if_ft must be 0 (none), 1 (checksums per group of tiles) or 2 (thread-level verification)"); return nullptr; }
    turbofft_plan* p = new turbofft_plan();
    p->logN = logN;
    p->datatype = datatype;
    p->if_err = if_err ? 1 : 0;
    p->if_ft = (if_ft || if_err) ? 1 : 0;            // CommandLineParser.h:66-68
    p->scheme = if_ft == 2 ? 1 : 0;
    p->thread_bs = thread_bs;
    if (p->if_err) { p->inj_mode = 1; p->correct = 1; }   // the if_err=1 kernels inject and correct
    const char* env = getenv("TURBOFFT_CHECKSUM_MODE");
    if (env && atoi(env) == 1) p->cksum_mode = 1;
    env = getenv("TURBOFFT_COMPACT_CHECKSUM");
    if (env && atoi(env) == 0) p->compact_enabled = false;
    env = getenv("TURBOFFT_XCD_CHUNK");
    if (env) p->xcd_chunk = atoi(env) > 0 ? atoi(env) : 0;
    if (plan_build(p, param_csv) != TURBOFFT_OK) {
        std::string keep = g_err;
        turbofft_plan_destroy(p);
        g_err = keep;
        return nullptr;
    }
    return p;
}

int turbofft_plan_info(const turbofft_plan_t* p, int* launches, int logNi[3], int BSi[3], int ni[3],
                       size_t lds_bytes[3], int threads[3]) {
    if (!p) return fail(TURBOFFT_EINVAL, "null plan");
    if (launches) *launches = p->launches;
    for (int i = 0; i < 3; ++i) {
        bool on = i < p->launches;
        if (logNi) logNi[i] = on ? p->row.logNi(i) : 0;
        if (BSi) BSi[i] = on ? p->row.BS(i) : 0;
        if (ni) ni[i] = on ? p->row.n(i) : 0;
        if (lds_bytes) lds_bytes[i] = on ? (size_t)p->k[i]->lds_bytes : 0;
        if (threads) threads[i] = on ? p->k[i]->threads : 0;
    }
    return TURBOFFT_OK;
}

static long long launch_tiles(const turbofft_plan* p, int i, long long bs) {
    long long tile = (1ll << p->row.logNi(i)) * p->row.BS(i);
    long long pts = (1ll << p->logN) * bs;
    if (p->launches == 1) return (bs + p->row.BS(0) - 1) / p->row.BS(0);
    return pts / tile;
}

// Tiles a block of launch i walks.  The row's tuned value was timed with the device full: a
// batch too small for that keeps at least one block per resident slot instead.
static int launch_thread_bs(const turbofft_plan* p, int i, long long ntiles) {
    if (!p->tiles_from_row) return p->thread_bs;
    long long per_slot = ntiles / (p->resident[i] > 0 ? p->resident[i] : 1);
    if (per_slot < 1) per_slot = 1;
    return per_slot < p->thread_bs ? (int)per_slot : p->thread_bs;
}

long long turbofft_plan_grid(const turbofft_plan_t* p, int launch, long long bs) {
    if (!p || launch < 0 || launch >= p->launches || bs < 0) return fail(TURBOFFT_EINVAL, "bad argument");
    long long nt = launch_tiles(p, launch, bs);
    int tbs = launch_thread_bs(p, launch, nt);
    return (nt + tbs - 1) / tbs;
}

int turbofft_plan_tb_gap(const turbofft_plan_t* p, int launch) {
    if (!p || launch < 0 || launch >= p->launches) return fail(TURBOFFT_EINVAL, "bad argument");
    return p->tb_gap[launch];
}

int turbofft_plan_set_tb_gap(turbofft_plan_t* p, int launch, int tb_gap) {
    if (!p || launch < 0 || launch >= p->launches || tb_gap < 1) return fail(TURBOFFT_EINVAL, "bad argument");
    p->tb_gap[launch] = tb_gap;
    return TURBOFFT_OK;
}

int turbofft_plan_set_ft_part_len(turbofft_plan_t* p, int launch, int tiles) {
    if (!p || launch < 0 || launch >= p->launches || tiles < 0) return fail(TURBOFFT_EINVAL, "bad argument");
    if (!p->if_ft) return fail(TURBOFFT_EINVAL, "plan was created without if_ft");
    p->ft_part_len[launch] = tiles;
    return TURBOFFT_OK;
}

int turbofft_plan_ft_part_len(const turbofft_plan_t* p, int launch) {
    if (!p || launch < 0 || launch >= p->launches) return 0;
    return p->ft_part_len[launch];
}

int turbofft_set_ft_params(turbofft_plan_t* p, double err_smoothing, double err_threshold, int correct) {
    if (!p) return fail(TURBOFFT_EINVAL, "null plan");
    if (!p->if_ft) return fail(TURBOFFT_EINVAL, "plan was created without if_ft");
    if (correct < 0 || correct > 2) return fail(TURBOFFT_EINVAL, "correct must be 0 (detect only), 1 (recompute) or 2 (delayed batch correction)");
    if (correct == 2 && p->scheme == 1) return fail(TURBOFFT_EINVAL, "thread-level verification recomputes a flagged tile before it is stored: correct is 0 or 1");
    if (correct == 2)
        for (int i = 0; i < p->launches; ++i)
            if (!p->k_dc[i])
                return fail(TURBOFFT_ENOPLAN, "no compiled delayed-correction kernel for launch %d of logN=%d (built for the built-in fault-tolerant plan rows)", i, p->logN);
    p->err_smoothing = err_smoothing;
    p->err_threshold = err_threshold;
    p->correct = correct;
    return TURBOFFT_OK;
}

int turbofft_set_injection(turbofft_plan_t* p, int mode, int launch, int every, long long tile_phase, int s,
                           int m, double mag) {
    if (!p) return fail(TURBOFFT_EINVAL, "null plan");
    if (!p->if_ft) return fail(TURBOFFT_EINVAL, "plan was created without if_ft");
    if (mode < 0 || mode > 2 || every < 1) return fail(TURBOFFT_EINVAL, "bad injection mode/every");
    int li = launch < 0 ? p->launches - 1 : launch;
    if (li >= p->launches) return fail(TURBOFFT_EINVAL, "bad injection launch");
    if (s < 0 || s >= p->row.BS(li) || m < 0 || m >= (1 << p->row.logNi(li)) / p->row.n(li))
        return fail(TURBOFFT_EINVAL, "injection element (s=%d, m=%d): need 0 <= s < BS=%d and 0 <= m < Ni/n=%d", s, m,
                    p->row.BS(li), (1 << p->row.logNi(li)) / p->row.n(li));
    if (mode == 2 && (tile_phase < 0 || tile_phase >= every)) return fail(TURBOFFT_EINVAL, "tile_phase must be in [0, every)");
    p->inj_mode = mode; p->inj_launch = launch; p->inj_every = every; p->inj_tile = tile_phase;
    p->inj_s = s; p->inj_m = m; p->inj_mag = mag;
    return TURBOFFT_OK;
}

// Wait for the work the counters depend on: the stream of the plan's most recent execution
// (other streams of the device keep running).  A stream handle that is no longer valid falls
// back to a device-wide wait.
static int sync_last_stream(turbofft_plan_t* p, hipStream_t* st_out) {
    hipStream_t st = (hipStream_t)p->last_stream.load(std::memory_order_acquire);
    hipError_t e = hipStreamSynchronize(st);
    if (e == hipErrorInvalidHandle || e == hipErrorContextIsDestroyed || e == hipErrorInvalidResourceHandle) {
        (void)hipGetLastError();
        st = nullptr;
        p->last_stream.store(nullptr, std::memory_order_release);
        e = hipDeviceSynchronize();
    }
    if (e != hipSuccess) return fail(TURBOFFT_EHIP, "waiting for the plan's last execution failed: %s", hipGetErrorString(e));
    *st_out = st;
    return TURBOFFT_OK;
}

int turbofft_reset_ft_counters(turbofft_plan_t* p) {
    if (!p) return fail(TURBOFFT_EINVAL, "null plan");
    if (!p->if_ft) return TURBOFFT_OK;
    hipStream_t st = nullptr;
    int rc = sync_last_stream(p, &st);
    if (rc) return rc;
    HIP_TRY(hipMemsetAsync(p->counters, 0, TFFT_FT_COUNTER_WORDS * sizeof(unsigned long long), st));
    HIP_TRY(hipMemsetAsync(p->flagged, 0xff, sizeof(long long) * 2 * p->flagged_cap, st));
    if (p->tickets) HIP_TRY(hipMemsetAsync(p->tickets, 0, sizeof(unsigned) * (size_t)p->tickets_n, st));
    if (p->fix_ctl) HIP_TRY(hipMemsetAsync(p->fix_ctl, 0, 2 * sizeof(unsigned), st));
    HIP_TRY(hipStreamSynchronize(st));
    return TURBOFFT_OK;
}

int turbofft_get_ft_counters(turbofft_plan_t* p, unsigned long long* checked, unsigned long long* detected,
                             unsigned long long* corrected, unsigned long long* uncorrectable,
                             long long* flagged, int cap, int* nflagged) {
    if (!p) return fail(TURBOFFT_EINVAL, "null plan");
    std::vector<unsigned long long> c(TFFT_FT_COUNTER_WORDS, 0ull);
    hipStream_t st = nullptr;
    if (p->if_ft) {
        int rc = sync_last_stream(p, &st);
        if (rc) return rc;
        HIP_TRY(hipMemcpyAsync(c.data(), p->counters, c.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost, st));
        HIP_TRY(hipStreamSynchronize(st));
    }
    // device counters: [0] checksum groups run (block 0 of every launch adds its grid size, so
    // replays of a captured graph count too); detections and detections that could not be located
    // are spread over 64 sub-counter lines; every located detection is corrected while
    // correction is switched on
    unsigned long long det = 0, unloc = 0;
    for (int k = 0; k < 64; ++k) {
        det += c[TFFT_FT_SUB0 + TFFT_FT_SUB_STRIDE * k];
        unloc += c[TFFT_FT_SUB0 + TFFT_FT_SUB_STRIDE * k + 1];
    }
    if (checked) *checked = c[0];
    if (detected) *detected = det;
    if (corrected) *corrected = p->correct ? det - unloc : 0;
    if (uncorrectable) *uncorrectable = unloc;
    int n = 0;
    if (flagged && cap > 0 && det > 0) {
        // every sub-counter line owns a 64th of the list; hand the recorded pairs out in line order
        const int region = p->flagged_cap / 64;
        std::vector<long long> all((size_t)2 * p->flagged_cap);
        HIP_TRY(hipMemcpyAsync(all.data(), p->flagged, all.size() * sizeof(long long), hipMemcpyDeviceToHost, st));
        HIP_TRY(hipStreamSynchronize(st));
        for (int k = 0; k < 64 && n < cap; ++k) {
            unsigned long long have = c[TFFT_FT_SUB0 + TFFT_FT_SUB_STRIDE * k];
            if (have > (unsigned long long)region) have = region;
            for (unsigned long long j = 0; j < have && n < cap; ++j, ++n) {
                flagged[2 * n] = all[2 * ((size_t)k * region + j)];
                flagged[2 * n + 1] = all[2 * ((size_t)k * region + j) + 1];
            }
        }
    }
    if (nflagged) *nflagged = n;
    return TURBOFFT_OK;
}

int turbofft_plan_set_small_batch(turbofft_plan_t* p, int enable) {
    if (!p) return fail(TURBOFFT_EINVAL, "null plan");
    p->small_enabled = enable != 0;
    return TURBOFFT_OK;
}

long long turbofft_plan_small_batch_max(const turbofft_plan_t* p) {
    if (!p) return fail(TURBOFFT_EINVAL, "null plan");
    return (p->small && p->small_enabled) ? p->small_max_bs : 0;
}

int turbofft_set_checksum_mode(turbofft_plan_t* p, int mode) {
    if (!p) return fail(TURBOFFT_EINVAL, "null plan");
    if (!p->if_ft) return fail(TURBOFFT_EINVAL, "plan was created without if_ft");
    if (mode != 0 && mode != 1) return fail(TURBOFFT_EINVAL, "checksum mode must be 0 (exact) or 1 (reference)");
    if (p->scheme == 1) return fail(TURBOFFT_EINVAL, "thread-level verification reads no checksum table (its vectors are constants of the kernels)");
    hipStream_t st = nullptr;
    int rc = sync_last_stream(p, &st);      // executions in flight still read the old tables
    if (rc) return rc;
    p->cksum_mode = mode;
    return upload_checksum_tables(p);
}

// ---- the library's static device workspace (turbofft_exec_static) --------------------------
// One array per GPU the library runs on, held until the process ends.  In host code the
// array's name is only a handle: the device address comes from hipGetSymbolAddress, once per
// device, and that pointer is what kernels and copies are given.
#define TFFT_STATIC_WS_BYTES TURBOFFT_STATIC_WORKSPACE_BYTES
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[TFFT_STATIC_WS_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// device address of `scratch` on the current device (looked up on first use per device)
int static_workspace(void** ptr) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(TURBOFFT_EINVAL, "device ordinal %d is beyond the %d this library tracks", dev, kMaxDevices);
    void* q = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!q) {
        hipError_t e = hipGetSymbolAddress(&q, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !q)
            return fail(TURBOFFT_EHIP, "hipGetSymbolAddress(static workspace) failed on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev].store(q, std::memory_order_release);
    }
    *ptr = q;
    return TURBOFFT_OK;
}
}  // namespace

struct exec_opts {
    hipEvent_t* ev = nullptr;     // launches+1 events: ev[i] before launch i, ev[launches] after the last
    bool inverse = false;
    bool sync_each = false;       // wait for every launch before issuing the next (the reference's timing loop)
    void* workspace = nullptr;    // non-null: N*bs elements of intermediate storage; `out` then holds N*bs only
    bool main_row = false;        // run the plan's own row whatever the batch (pieces of a larger batch)
    void* pair_ws = nullptr;      // set for the plan of a fused pair: the turbofft_plan::PairWs to run it with
};

static int exec_impl(turbofft_plan_t* p, const void* in_d, void* out_d, long long bs, void* stream, const exec_opts& o);

int turbofft_exec(turbofft_plan_t* p, const void* in_d, void* out_d, long long bs, void* stream) {
    return exec_impl(p, in_d, out_d, bs, stream, exec_opts());
}

int turbofft_exec_inverse(turbofft_plan_t* p, const void* in_d, void* out_d, long long bs, void* stream) {
    exec_opts o;
    o.inverse = true;
    return exec_impl(p, in_d, out_d, bs, stream, o);
}

int turbofft_exec_static(turbofft_plan_t* p, const void* in_d, void* out_d, long long bs, void* stream) {
    if (!p) return fail(TURBOFFT_EINVAL, "null plan");
    if (bs < 0) return fail(TURBOFFT_EINVAL, "negative batch");
    exec_opts o;
    const bool small = p->small && p->small_enabled && bs <= p->small_max_bs;
    if (p->launches > 1 || small) {
        // the intermediate of a multi-launch plan is N*bs elements
        const unsigned long long need = ((unsigned long long)bs << p->logN) * p->esize;
        if ((bs >> (62 - p->logN)) != 0 || need > TFFT_STATIC_WS_BYTES)
            return fail(TURBOFFT_EINVAL, "turbofft_exec_static: %lld transforms of 2^%d points need %llu bytes of intermediate "
                        "storage, the static workspace holds %llu; use turbofft_exec with a 2*N*bs output buffer",
                        bs, p->logN, need, (unsigned long long)TFFT_STATIC_WS_BYTES);
        int rc = static_workspace(&o.workspace);
        if (rc) return rc;
    }
    return exec_impl(p, in_d, out_d, bs, stream, o);
}

// the kernel launch i runs with the plan's current settings
static const tfft_kernel_entry* launch_kernel(const turbofft_plan* p, int i, bool inverse) {
    const tfft_kernel_entry* k = inverse ? p->k_inv[i] : (p->correct == 2 ? p->k_dc[i] : p->k[i]);
    // The compact checksum table holds exact-angle entries in reduced precision: tighter
    // detection rules and the reference's own table run the full-table flavour of the launch.
    if (k && k->ck && (p->cksum_mode != 0 || !p->compact_enabled ||
                       p->err_threshold < (p->datatype == TURBOFFT_FP32 ? kCompactMinThreshold32 : kCompactMinThreshold64))) k = p->k_full[i];
    return k;
}

const char* turbofft_plan_kernel_name(const turbofft_plan_t* p, int launch) {
    if (!p || launch < 0 || launch >= p->launches) { fail(TURBOFFT_EINVAL, "bad argument"); return nullptr; }
    const tfft_kernel_entry* k = launch_kernel(p, launch, false);
    return k ? k->name : nullptr;
}

// true while `stream` records into a HIP graph: nothing may be allocated or cleared from the host then
static bool stream_is_capturing(void* stream) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t)stream, &st) != hipSuccess) { (void)hipGetLastError(); return false; }
    return st != hipStreamCaptureStatusNone;
}

// Slots, tickets and queue of checksum groups shared by several blocks: allocated by the first
// execution that needs them (128 MiB + 12 MiB a plan with short groups, or one that only ever runs
// small batches, never pays for).  Returns false when they are absent and cannot be made now (the
// stream is being captured, or the allocation failed): the execution then walks whole groups.
static bool ensure_part_slots(turbofft_plan* p, void* stream) {
    if (p->part_sums) return true;
    if (stream_is_capturing(stream)) return false;
    void *ps = nullptr, *tk = nullptr, *fl = nullptr, *fc = nullptr;
    const size_t tn = (size_t)kPartTickets;
    bool ok = hipMalloc(&ps, kPartSumsBytes) == hipSuccess && hipMalloc(&tk, sizeof(unsigned) * tn) == hipSuccess &&
              hipMalloc(&fl, sizeof(long long) * tn) == hipSuccess && hipMalloc(&fc, 2 * sizeof(unsigned)) == hipSuccess;
    // cleared on the stream the execution is issued on, ahead of its kernels
    ok = ok && hipMemsetAsync(tk, 0, sizeof(unsigned) * tn, (hipStream_t)stream) == hipSuccess &&
         hipMemsetAsync(fc, 0, 2 * sizeof(unsigned), (hipStream_t)stream) == hipSuccess;
    if (!ok) {
        (void)hipGetLastError();
        if (ps) (void)hipFree(ps);
        if (tk) (void)hipFree(tk);
        if (fl) (void)hipFree(fl);
        if (fc) (void)hipFree(fc);
        return false;
    }
    p->part_sums = ps; p->tickets = (unsigned*)tk; p->fix_list = (long long*)fl; p->fix_ctl = (unsigned*)fc;
    p->part_sums_bytes = kPartSumsBytes;
    p->tickets_n = kPartTickets;
    return true;
}

// The row a batch of `bs` transforms runs: the small-batch row (plain built-in plans, bs up to its cap), the fused
// pair (batches that give every team a piece) or the plan's own
static const turbofft_plan* row_for_batch(const turbofft_plan* p, long long bs) {
    if (p->small && p->small_enabled && bs >= 1 && bs <= p->small_max_bs) return p->small;
    if (p->pair && p->pair_enabled && (bs + p->pair->pair_per_piece - 1) / p->pair->pair_per_piece >= 8ll * p->pair->pair_teams_per_xcd) return p->pair;
    return p;
}

int turbofft_plan_launches_for_batch(const turbofft_plan_t* p, long long bs) {
    if (!p || bs < 0) return fail(TURBOFFT_EINVAL, "bad argument");
    const turbofft_plan* q = row_for_batch(p, bs);
    return q->pk ? 1 : q->launches;
}

const char* turbofft_plan_kernel_name_for_batch(const turbofft_plan_t* p, int launch, long long bs) {
    if (!p || bs < 0) { fail(TURBOFFT_EINVAL, "bad argument"); return nullptr; }
    const turbofft_plan* q = row_for_batch(p, bs);
    if (launch < 0 || launch >= (q->pk ? 1 : q->launches)) { fail(TURBOFFT_EINVAL, "bad argument"); return nullptr; }
    if (q->pk) return q->pk->name;
    const tfft_kernel_entry* k = launch_kernel(q, launch, false);
    return k ? k->name : nullptr;
}

int turbofft_plan_set_fused(turbofft_plan_t* p, int enable) {
    if (!p) return fail(TURBOFFT_EINVAL, "null plan");
    if (enable && !p->pair) return fail(TURBOFFT_ENOPLAN, "the plan holds no fused kernel (none for this size, or created without TURBOFFT_FUSED=1)");
    p->pair_enabled = enable != 0;
    return TURBOFFT_OK;
}

int turbofft_plan_fused_info(const turbofft_plan_t* p, int* team_blocks, int* transforms_per_piece, int* teams_per_xcd, int* grid_blocks) {
    if (!p) return fail(TURBOFFT_EINVAL, "null plan");
    const turbofft_plan* q = p->pair;
    if (team_blocks) *team_blocks = q ? q->pair_team : 0;
    if (transforms_per_piece) *transforms_per_piece = q ? q->pair_per_piece : 0;
    if (teams_per_xcd) *teams_per_xcd = q ? q->pair_teams_per_xcd : 0;
    if (grid_blocks) *grid_blocks = q ? q->pair_grid : 0;
    return (q && p->pair_enabled) ? 1 : 0;
}

static bool ranges_overlap(const void* a, size_t an, const void* b, size_t bn) {
    const char *a0 = (const char*)a, *b0 = (const char*)b;
    return a0 < b0 + bn && b0 < a0 + an;
}

static int exec_impl(turbofft_plan_t* p, const void* in_d, void* out_d, long long bs, void* stream, const exec_opts& o) {
    if (!p) return fail(TURBOFFT_EINVAL, "null plan");
    const bool inverse = o.inverse;
    if (inverse) {
        if (p->if_ft) return fail(TURBOFFT_ENOPLAN, "fault-tolerant plans have no inverse kernels");
        for (int i = 0; i < p->launches; ++i)
            if (!p->k_inv[i])
                return fail(TURBOFFT_ENOPLAN, "no compiled inverse kernel for launch %d of logN=%d (built for the built-in plan rows only)", i, p->logN);
    }
    if (bs < 0) return fail(TURBOFFT_EINVAL, "negative batch");
    if (bs == 0) return TURBOFFT_OK;
    if (!in_d || !out_d) return fail(TURBOFFT_EINVAL, "null buffer");
    const long long N = 1ll << p->logN;
    if (N * bs > (1ll << 40)) return fail(TURBOFFT_EINVAL, "problem too large");
    const size_t data_bytes = (size_t)N * bs * p->esize;
    char* out = (char*)out_d;
    if (p->small && p->small_enabled && bs <= p->small_max_bs && !inverse && !o.main_row) {
        // few transforms: the narrow-tile row, with the caller's workspace half when there is
        // one, else the plan's own intermediate buffer
        exec_opts so = o;
        bool have_ws = true;
        if (!so.workspace && p->launches == 1) {
            // the intermediate of the two narrow-tile launches: a buffer of the plan's, one per stream, so that
            // executions of one plan on several streams do not share it.  A stream without one gets one now,
            // unless it is being captured or the plan already keeps kMaxSmallWs: then the main row runs.
            std::lock_guard<std::mutex> lk(p->small_mu);
            turbofft_plan::SmallWs* w = nullptr;
            for (auto& e : p->small_ws) if (e.assigned && e.stream == stream) { w = &e; break; }
            if (!w) for (auto& e : p->small_ws) if (!e.assigned) { e.assigned = true; e.stream = stream; w = &e; break; }
            if (!w && p->small_ws.size() < kMaxSmallWs && !stream_is_capturing(stream)) {
                void* buf = nullptr;
                if (hipMalloc(&buf, ((size_t)p->small_max_bs << p->logN) * p->esize) == hipSuccess) {
                    p->small_ws.push_back({stream, true, buf});
                    w = &p->small_ws.back();
                } else {
                    (void)hipGetLastError();
                }
            }
            if (w) so.workspace = w->buf; else have_ws = false;
        }
        if (have_ws) {
        if (ranges_overlap(in_d, data_bytes, out, data_bytes * ((p->launches > 1 && !o.workspace) ? 2 : 1)))
            return fail(TURBOFFT_EINVAL, "in [%p, +%zu) overlaps out [%p, ...): the transform is out of place", in_d, data_bytes, (void*)out);
        p->last_stream.store(stream, std::memory_order_release);
        return exec_impl(p->small, in_d, out_d, bs, stream, so);
        }
    }
    if (p->pair && p->pair_enabled && !inverse && !o.main_row && !o.ev &&
        (bs + p->pair->pair_per_piece - 1) / p->pair->pair_per_piece >= 8ll * p->pair->pair_teams_per_xcd) {
        // both launches as one kernel, where every team gets at least one piece: the slots and control block of this
        // stream (a stream without a set gets one now, unless it is being captured or the plan keeps kMaxPairWs
        // already: then the two launches run)
        turbofft_plan::PairWs* w = nullptr;
        {
            std::lock_guard<std::mutex> lk(p->pair_mu);
            for (auto& e : p->pair_ws) if (e.assigned && e.stream == stream) { w = &e; break; }
            if (!w) for (auto& e : p->pair_ws) if (!e.assigned) { e.assigned = true; e.stream = stream; w = &e; break; }
            // (a caller that brought its own workspace may be one that cannot allocate: no new set for it)
            if (!w && !o.workspace && p->pair_ws.size() < kMaxPairWs && !stream_is_capturing(stream) && pair_add_ws(p, p->pair, stream, true)) w = &p->pair_ws.back();
        }
        if (w) {
            if (*(volatile unsigned*)w->err_host) {
                // an earlier execution on this stream gave up waiting (its blocks were not all resident in time):
                // what it left in `out` is incomplete.  The plan goes back to its two launches.
                *(volatile unsigned*)w->err_host = 0u;
                p->pair_enabled = false;
                return fail(TURBOFFT_EHIP, "an earlier execution of the fused kernel of this plan ran out of time waiting for its blocks to be "
                            "resident together; its output is incomplete.  The plan runs its two launches from now on");
            }
            if (ranges_overlap(in_d, data_bytes, out, data_bytes))
                return fail(TURBOFFT_EINVAL, "in [%p, +%zu) overlaps out [%p, ...): the transform is out of place", in_d, data_bytes, (void*)out);
            p->last_stream.store(stream, std::memory_order_release);
            exec_opts po = o;
            po.pair_ws = w;
            return exec_impl(p->pair, in_d, out_d, bs, stream, po);
        }
    }
    const Row& r = p->row;
    char* work = o.workspace ? (char*)o.workspace : out + data_bytes;
    // The transform is out of place: the kernels read `in` while they write `out` (and a
    // fault-tolerant plan reads a located tile a second time), and the workspace half of `out`
    // is overwritten by the first launch of a multi-launch plan.
    const size_t out_bytes = data_bytes * ((p->launches > 1 && !o.workspace) ? 2 : 1);
    if (ranges_overlap(in_d, data_bytes, out, out_bytes))
        return fail(TURBOFFT_EINVAL, "in [%p, +%zu) overlaps out [%p, +%zu): the transform is out of place%s", in_d, data_bytes,
                    (void*)out, out_bytes, p->launches > 1 && !o.workspace ? " and out holds 2*N*bs elements (result + workspace)" : "");
    if (o.workspace && (ranges_overlap(in_d, data_bytes, work, data_bytes) || ranges_overlap(out, data_bytes, work, data_bytes)))
        return fail(TURBOFFT_EINVAL, "a buffer overlaps the workspace");
    // ping-pong so that the last launch writes out[0 .. N*bs)
    const void* src[3];
    void* dst[3];
    if (p->launches == 1) { src[0] = in_d; dst[0] = out; }
    else if (p->launches == 2) { src[0] = in_d; dst[0] = work; src[1] = work; dst[1] = out; }
    else { src[0] = in_d; dst[0] = out; src[1] = out; dst[1] = work; src[2] = work; dst[2] = out; }
    p->last_stream.store(stream, std::memory_order_release);
    tfft_kargs pair_args[2];
    for (int i = 0; i < p->launches; ++i) {
        const tfft_kernel_entry* k = launch_kernel(p, i, inverse);
        tfft_kargs a;
        memset(&a, 0, sizeof a);
        a.ntiles = launch_tiles(p, i, bs);
        a.nrows = bs;
        a.thread_bs = launch_thread_bs(p, i, a.ntiles);
        a.tb_gap = p->tb_gap[i];
        if (k->pf && !p->if_ft && p->thread_bs == 1 && a.ntiles > p->resident[i]) {
            // prefetching kernels run as a persistent grid: one block per resident slot walks
            // the tiles with the grid as stride, so there is always a next tile to fetch
            a.tb_gap = p->resident[i];
            a.thread_bs = (int)((a.ntiles + p->resident[i] - 1) / p->resident[i]);
        }
        a.xcd_chunk = p->xcd_chunk >= 0 ? p->xcd_chunk : p->xcd_chunk_l[i];
        int kind = kind_of_launch(p->launches, i);
        if (kind == 1) {
            int log_ncols = 0;
            for (int j = i + 1; j < p->launches; ++j) log_ncols += r.logNi(j);
            a.log_ncols = log_ncols;
            a.tw_lo_bits = p->lo_bits[i];
            int L = r.logNi(i) + log_ncols;
            long long hiN = 1ll << (L - p->lo_bits[i]);
            a.tw_hi = (const char*)p->tw + (size_t)(hiN - 1) * p->esize;
            a.tw_lo = p->tw_lo[i];
        } else if (kind == 2) {
            a.logN = p->logN;
            a.logC = r.logNi(0);
            a.logQ = p->launches == 3 ? r.logNi(1) : 0;
        }
        if (p->if_ft) {
            a.ft.cksum = p->scheme == 1 ? nullptr : (k->ck ? p->cksum16[i] : p->cksum[i]);
            a.ft.counters = p->counters;
            a.ft.flagged = p->flagged;
            a.ft.flagged_cap = p->flagged_cap;
            a.ft.launch = i;
            a.ft.correct = p->correct ? 1 : 0;
            int inj_l = p->inj_launch < 0 ? p->launches - 1 : p->inj_launch;
            a.ft.inj_mode = (inj_l == i) ? p->inj_mode : 0;
            a.ft.inj_every = p->inj_every;
            a.ft.inj_tile = p->inj_tile;
            a.ft.inj_s = p->inj_s;
            a.ft.inj_m = p->inj_m;
            a.ft.inj_mag = p->inj_mag;
            a.ft.err_smoothing = p->err_smoothing;
            a.ft.err_threshold = p->err_threshold;
        }
        if (o.pair_ws) { pair_args[i] = a; continue; }     // the fused kernel takes both launches' arguments
        long long grid = (a.ntiles + a.thread_bs - 1) / a.thread_bs;
        if (grid < 1) continue;
        long long fix_grid = 0;
        if (p->if_ft && k->ft == 1 && !k->pf && p->ft_part_len[i] > 0 && a.thread_bs > p->ft_part_len[i]) {
            // groups longer than ft_part_len tiles: several blocks per group, where the plan's slots suffice
            const long long parts = (a.thread_bs + p->ft_part_len[i] - 1) / p->ft_part_len[i];
            const unsigned long long need = (unsigned long long)grid * parts * 4ull * k->threads * (p->esize / 2);
            if (need <= kPartSumsBytes && grid <= kPartTickets && grid * parts <= 0x7fffffffll && ensure_part_slots(p, stream)) {
                a.ft.parts = (int)parts;
                a.ft.part_len = p->ft_part_len[i];
                a.ft.part_sums = p->part_sums;
                a.ft.tickets = p->tickets;
                a.ft.fix_list = p->fix_list;
                a.ft.fix_ctl = p->fix_ctl;
                if (a.ft.correct) fix_grid = grid < kFixGrid ? grid : kFixGrid;
                grid *= parts;
            }
        }
        if (grid > 0x7fffffffll) return fail(TURBOFFT_EINVAL, "grid of %lld blocks exceeds the launch limit", grid);
        const void* in_arg = src[i];
        void* out_arg = dst[i];
        const void* tw_arg = p->tw;
        void* args[4] = {(void*)&in_arg, (void*)&out_arg, (void*)&tw_arg, (void*)&a};
        if (o.ev) HIP_TRY(hipEventRecord(o.ev[i], (hipStream_t)stream));
        HIP_TRY(hipLaunchKernel(k->func, dim3((unsigned)grid), dim3((unsigned)k->threads), args, (size_t)k->lds_bytes,
                                (hipStream_t)stream));
        if (fix_grid) {
            // groups shared by several blocks: tiles found wrong are recomputed by a second launch of
            // the same kernel (a kernel boundary orders the two stores of such a tile, which come
            // from blocks on different XCDs); with nothing queued its blocks return at once
            a.ft.parts = 1;
            a.ft.fix_mode = 1;
            HIP_TRY(hipLaunchKernel(k->func, dim3((unsigned)fix_grid), dim3((unsigned)k->threads), args, (size_t)k->lds_bytes,
                                    (hipStream_t)stream));
        }
        if (o.sync_each) HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    }
    if (o.pair_ws) {
        const turbofft_plan::PairWs* w = (const turbofft_plan::PairWs*)o.pair_ws;
        tfft_fuse_args f;
        memset(&f, 0, sizeof f);
        f.slots = w->slots;
        f.ctl = w->ctl;
        f.err_host = w->err_host;
        f.piece_elems = (long long)p->pair_per_piece << p->logN;
        f.npieces = (bs + p->pair_per_piece - 1) / p->pair_per_piece;
        f.tiles_a = p->pair_per_piece * ((1 << r.logNi(1)) / r.BS(0));
        f.tiles_b = p->pair_per_piece * ((1 << r.logNi(0)) / r.BS(1));
        f.team = p->pair_team;
        f.teams_per_xcd = p->pair_teams_per_xcd;
        f.limit_ms = p->pair_limit_ms;
        f.prof = w->prof;          // diagnostic builds of the kernel only (TFFT_PAIR_PROFILE at build time) write it
        if (f.npieces > 0x7fffffffll) return fail(TURBOFFT_EINVAL, "too many pieces for the fused kernel");
        const void* in_arg = in_d;
        void* out_arg = out;
        const void* tw_arg = p->tw;
        void* args[6] = {(void*)&in_arg, (void*)&out_arg, (void*)&tw_arg, (void*)&pair_args[0], (void*)&pair_args[1], (void*)&f};
        HIP_TRY(hipLaunchKernel(p->pk->func, dim3((unsigned)p->pair_grid), dim3((unsigned)p->pk->threads), args, (size_t)p->pk->lds_bytes,
                                (hipStream_t)stream));
        if (o.sync_each) HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
        if (f.prof && !stream_is_capturing(stream)) {
            // TURBOFFT_FUSED_PROF=1 when the plan was made: wait for the execution and print what a diagnostic build of the
            // kernel timed (ticks of 10 ns per block and part of a round; all zero from a product build)
            HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
            std::vector<unsigned long long> h((size_t)8 * p->pair_grid);
            HIP_TRY(hipMemcpy(h.data(), f.prof, h.size() * 8, hipMemcpyDeviceToHost));
            double t[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int b = 0; b < p->pair_grid; ++b) for (int k = 0; k < 8; ++k) t[k] += (double)h[8 * b + k];
            const double rounds = t[4] > 0 ? t[4] : 1;
            fprintf(stderr, "fused %s: per round, us: column launch %.2f, meeting %.2f, row launch: slot loads %.2f, first phase %.2f, fetch ahead %.2f, rest %.2f, slot wait %.2f (%.1f rounds per block)\n",
                    p->pk->name, t[0] / rounds / 100, t[1] / rounds / 100, t[7] / rounds / 100, t[5] / rounds / 100, t[6] / rounds / 100, t[2] / rounds / 100, t[3] / rounds / 100, t[4] / p->pair_grid);
        }
        return TURBOFFT_OK;
    }
    if (o.ev) HIP_TRY(hipEventRecord(o.ev[p->launches], (hipStream_t)stream));
    return TURBOFFT_OK;
}

namespace {
// events that are destroyed on every way out of a timing function
struct EventSet {
    std::vector<hipEvent_t> ev;
    int create(int n) {
        for (int i = 0; i < n; ++i) {
            hipEvent_t e;
            HIP_TRY(hipEventCreate(&e));
            ev.push_back(e);
        }
        return TURBOFFT_OK;
    }
    ~EventSet() { for (hipEvent_t e : ev) (void)hipEventDestroy(e); }
};
}  // namespace

int turbofft_time_launches(turbofft_plan_t* p, const void* in_d, void* out_d, long long bs, int warmup, int reps,
                           void* stream, float ms_per_launch[3]) {
    if (!p || !ms_per_launch || reps < 1 || warmup < 0 || bs < 1) return fail(TURBOFFT_EINVAL, "bad argument");
    for (int i = 0; i < 3; ++i) ms_per_launch[i] = 0.f;
    for (int i = 0; i < warmup; ++i) {
        exec_opts wo;
        wo.main_row = true;
        int rc = exec_impl(p, in_d, out_d, bs, stream, wo);
        if (rc) return rc;
    }
    EventSet es;
    int rc = es.create(4);
    if (rc) return rc;
    exec_opts o;
    o.ev = es.ev.data();
    o.main_row = true;          // the plan's own row whatever the batch: its launches are what the caller gets times for
    for (int r = 0; r < reps; ++r) {
        rc = exec_impl(p, in_d, out_d, bs, stream, o);
        if (rc) return rc;
        HIP_TRY(hipEventSynchronize(es.ev[p->launches]));
        for (int i = 0; i < p->launches; ++i) {
            float ms = 0;
            HIP_TRY(hipEventElapsedTime(&ms, es.ev[i], es.ev[i + 1]));
            ms_per_launch[i] += ms / reps;
        }
    }
    return TURBOFFT_OK;
}

namespace {
// device buffers, streams and events of one host-buffer execution, released on every way out
struct HostPipe {
    turbofft_plan_t* plan = nullptr;       // its last-execution stream must not outlive the streams below
    std::vector<void*> dev;
    std::vector<hipStream_t> st;
    EventSet ev;
    int alloc(void** q, size_t bytes) {
        if (hipMalloc(q, bytes) != hipSuccess) { (void)hipGetLastError(); return fail(TURBOFFT_ENOMEM, "hipMalloc(%zu) failed", bytes); }
        dev.push_back(*q);
        return TURBOFFT_OK;
    }
    int stream(hipStream_t* q) {
        HIP_TRY(hipStreamCreateWithFlags(q, hipStreamNonBlocking));
        st.push_back(*q);
        return TURBOFFT_OK;
    }
    ~HostPipe() {
        for (hipStream_t q : st) (void)hipStreamSynchronize(q);   // nothing may still use the buffers
        if (plan && !st.empty()) plan->last_stream.store(nullptr, std::memory_order_release);
        for (hipStream_t q : st) (void)hipStreamDestroy(q);
        for (void* q : dev) (void)hipFree(q);
    }
};

// Transforms the whole batch in one piece: the path of fault-tolerant plans (their tile groups
// and the tile numbers of the flagged list refer to the batch as the caller passed it) and of
// batches that are a single piece anyway.
int exec_host_whole(turbofft_plan_t* p, const void* in_h, void* out_h, long long bs, size_t bytes) {
    HostPipe hp;
    void *in_d = nullptr, *out_d = nullptr;
    int rc = hp.alloc(&in_d, bytes);
    if (rc) return rc;
    rc = hp.alloc(&out_d, bytes * (p->launches > 1 ? 2 : 1));
    if (rc) return rc;
    HIP_TRY(hipMemcpy(in_d, in_h, bytes, hipMemcpyHostToDevice));
    rc = turbofft_exec(p, in_d, out_d, bs, nullptr);
    if (rc) return rc;
    HIP_TRY(hipStreamSynchronize(nullptr));
    HIP_TRY(hipMemcpy(out_h, out_d, bytes, hipMemcpyDeviceToHost));
    return TURBOFFT_OK;
}

size_t host_piece_bytes() {
    // bytes of input one piece of the streamed host path carries (TURBOFFT_HOST_PIECE_BYTES overrides)
    if (const char* e = std::getenv("TURBOFFT_HOST_PIECE_BYTES")) {
        long long v = std::atoll(e);
        if (v > 0) return (size_t)v;
    }
    return (size_t)64 << 20;       // timed 32-256 MiB with page-locked buffers: 64 MiB pieces were fastest
}
}  // namespace

int turbofft_exec_host(turbofft_plan_t* p, const void* in_h, void* out_h, long long bs) {
    if (!p) return fail(TURBOFFT_EINVAL, "null plan");
    if (bs < 0) return fail(TURBOFFT_EINVAL, "negative batch");
    if (bs == 0) return TURBOFFT_OK;
    if (!in_h || !out_h) return fail(TURBOFFT_EINVAL, "null buffer");
    const size_t one = ((size_t)1 << p->logN) * p->esize;            // bytes of one transform
    const size_t bytes = one * (size_t)bs;
    long long piece = (long long)(host_piece_bytes() / one);
    if (piece < 1) piece = 1;
    if (p->if_ft || p->if_err || piece >= bs) return exec_host_whole(p, in_h, out_h, bs, bytes);

    // Plain plan, several pieces: the batch streams through three slots of device memory.
    // One stream copies pieces in, one runs the plan on them in order (so nothing the plan
    // owns is used by two executions at once), one copies results out; events hand a slot
    // from stage to stage.  With page-locked host buffers the two copy directions and the
    // kernels overlap; pageable buffers make each copy call block the host, which still
    // bounds the device memory to the three slots.
    const int kSlots = 3;
    const long long pieces = (bs + piece - 1) / piece;
    const int slots = pieces < kSlots ? (int)pieces : kSlots;
    const size_t pbytes = one * (size_t)piece;
    HostPipe hp;
    hp.plan = p;
    hipStream_t s_in, s_run, s_out;
    int rc;
    if ((rc = hp.stream(&s_in)) || (rc = hp.stream(&s_run)) || (rc = hp.stream(&s_out))) return rc;
    void *in_d[kSlots] = {}, *out_d[kSlots] = {};
    for (int i = 0; i < slots; ++i) {
        if ((rc = hp.alloc(&in_d[i], pbytes))) return rc;
        if ((rc = hp.alloc(&out_d[i], pbytes * (p->launches > 1 ? 2 : 1)))) return rc;
    }
    if ((rc = hp.ev.create(3 * slots))) return rc;
    hipEvent_t* copied = hp.ev.ev.data();                              // piece is in in_d[slot]
    hipEvent_t* ran = copied + slots;                                  // in_d[slot] consumed, out_d[slot] holds the result
    hipEvent_t* drained = ran + slots;                                 // out_d[slot] is on the host
    exec_opts eo;
    // every piece runs the kernels the whole batch would run on the device path: the same bits
    eo.main_row = !(p->small && p->small_enabled && bs <= p->small_max_bs);
    for (long long c = 0; c < pieces; ++c) {
        const int k = (int)(c % slots);
        const long long b0 = c * piece, nb = (bs - b0 < piece) ? bs - b0 : piece;
        const char* src = (const char*)in_h + (size_t)b0 * one;
        char* dst = (char*)out_h + (size_t)b0 * one;
        if (c >= slots) HIP_TRY(hipStreamWaitEvent(s_in, ran[k], 0));
        HIP_TRY(hipMemcpyAsync(in_d[k], src, one * (size_t)nb, hipMemcpyHostToDevice, s_in));
        HIP_TRY(hipEventRecord(copied[k], s_in));
        HIP_TRY(hipStreamWaitEvent(s_run, copied[k], 0));
        if (c >= slots) HIP_TRY(hipStreamWaitEvent(s_run, drained[k], 0));
        if ((rc = exec_impl(p, in_d[k], out_d[k], nb, s_run, eo))) return rc;
        HIP_TRY(hipEventRecord(ran[k], s_run));
        HIP_TRY(hipStreamWaitEvent(s_out, ran[k], 0));
        HIP_TRY(hipMemcpyAsync(dst, out_d[k], one * (size_t)nb, hipMemcpyDeviceToHost, s_out));
        HIP_TRY(hipEventRecord(drained[k], s_out));
    }
    HIP_TRY(hipStreamSynchronize(s_out));
    return TURBOFFT_OK;
}

static int time_impl(turbofft_plan_t* p, const void* in_d, void* out_d, long long bs, int warmup, int reps,
                     void* stream, float* ms_per_exec, bool sync_each) {
    if (!p || !ms_per_exec || reps < 1 || warmup < 0) return fail(TURBOFFT_EINVAL, "bad argument");
    hipStream_t st = (hipStream_t)stream;
    exec_opts o;
    o.sync_each = sync_each;
    for (int i = 0; i < warmup; ++i) {
        int rc = exec_impl(p, in_d, out_d, bs, stream, o);
        if (rc) return rc;
    }
    EventSet es;
    int rc = es.create(2);
    if (rc) return rc;
    HIP_TRY(hipEventRecord(es.ev[0], st));
    for (int i = 0; i < reps; ++i) {
        rc = exec_impl(p, in_d, out_d, bs, stream, o);
        if (rc) return rc;
        if (sync_each) HIP_TRY(hipStreamSynchronize(st));      // main.cu:61
    }
    HIP_TRY(hipEventRecord(es.ev[1], st));
    HIP_TRY(hipEventSynchronize(es.ev[1]));
    float ms = 0;
    HIP_TRY(hipEventElapsedTime(&ms, es.ev[0], es.ev[1]));
    *ms_per_exec = ms / reps;
    return TURBOFFT_OK;
}

int turbofft_time(turbofft_plan_t* p, const void* in_d, void* out_d, long long bs, int warmup, int reps,
                  void* stream, float* ms_per_exec) {
    return time_impl(p, in_d, out_d, bs, warmup, reps, stream, ms_per_exec, false);
}

int turbofft_time_sync(turbofft_plan_t* p, const void* in_d, void* out_d, long long bs, int warmup, int reps,
                       void* stream, float* ms_per_exec) {
    return time_impl(p, in_d, out_d, bs, warmup, reps, stream, ms_per_exec, true);
}

}  // extern "C"
