// Walks every host-side path of the library that needs no device: table builders, plan
// rows, plan CSV parsing (well formed and malformed), argument checks of the entry points,
// the command line.  Built with the host sources under AddressSanitizer and
// UndefinedBehaviorSanitizer by tests/test_host_sanitized.py; exits non-zero on a wrong answer.
#include <cstdio>
#include <initializer_list>
#include <vector>

#include "turbofft.h"

#define EXPECT(cond)                                                    \
    do {                                                                \
        if (!(cond)) {                                                  \
            std::printf("FAILED line %d: %s\n", __LINE__, #cond);       \
            return 1;                                                   \
        }                                                               \
    } while (0)

int main(int argc, char** argv) {
    std::vector<double> buf(2 * 2 * 8192);
    for (int dt = 0; dt < 2; ++dt) {
        for (long long N : {1ll, 2ll, 64ll, 8192ll}) EXPECT(turbofft_build_twiddle_table(dt, N, buf.data()) == 0);
        for (long long N : {2ll, 64ll, 1024ll})
            for (int mode = 0; mode < 2; ++mode) EXPECT(turbofft_build_checksum_vector(dt, N, mode, buf.data()) == 0);
        int row[11];
        for (int L = 1; L < 30; ++L) EXPECT(turbofft_builtin_plan_row(dt, L, row) == 0);
        EXPECT(turbofft_builtin_plan_row(dt, 40, row) != 0);
        EXPECT(turbofft_builtin_plan_row(dt, -1, row) != 0);
    }
    EXPECT(turbofft_build_twiddle_table(0, 3, buf.data()) != 0);
    EXPECT(turbofft_build_twiddle_table(7, 8, buf.data()) != 0);
    EXPECT(turbofft_build_checksum_vector(0, 8, 7, buf.data()) != 0);

    // the built-in table is parsed before a device is looked for: without one the plan fails cleanly
    for (int dt = 0; dt < 2; ++dt)
        for (int L : {0, 1, 13, 24, 29, 30, -3})
            for (int ft = 0; ft < 2; ++ft) {
                turbofft_plan_t* p = turbofft_plan_create(L, dt, ft, 0, 1, nullptr);
                if (p) turbofft_plan_destroy(p);          // (a machine with a GPU)
                else EXPECT(turbofft_last_error()[0] != 0);
            }
    // plan CSVs named on the command line: every one is malformed or describes shapes no kernel has
    for (int i = 1; i < argc; ++i)
        for (int dt = 0; dt < 2; ++dt)
            for (int L : {0, 5, 10, 29})
                for (int ft = 0; ft < 2; ++ft) {
                    turbofft_plan_t* p = turbofft_plan_create(L, dt, ft, 0, 1, argv[i]);
                    EXPECT(p == nullptr);
                    EXPECT(turbofft_last_error()[0] != 0);
                }
    EXPECT(turbofft_plan_create(10, 0, 0, 0, 1, "/nonexistent/plan.csv") == nullptr);

    EXPECT(turbofft_exec(nullptr, nullptr, nullptr, 1, nullptr) != 0);
    EXPECT(turbofft_exec_inverse(nullptr, nullptr, nullptr, 1, nullptr) != 0);
    EXPECT(turbofft_exec_static(nullptr, nullptr, nullptr, 1, nullptr) != 0);
    EXPECT(turbofft_exec_host(nullptr, nullptr, nullptr, 1) != 0);
    turbofft_plan_destroy(nullptr);

    int n = turbofft_kernel_count();
    EXPECT(n > 0);
    for (int i = 0; i < n; ++i) EXPECT(turbofft_kernel_name(i) != nullptr);
    EXPECT(turbofft_kernel_name(n) == nullptr);
    EXPECT(turbofft_kernel_name(-1) == nullptr);

    char a0[] = "turbofft", h[] = "--help", b1[] = "--bogus", b2[] = "1", l[] = "--logN";
    char* help[] = {a0, h};
    turbofft_main(2, help);
    char* bogus[] = {a0, b1, b2};
    EXPECT(turbofft_main(3, bogus) != 0);
    char* dangling[] = {a0, l};                           // option without its value
    EXPECT(turbofft_main(2, dangling) != 0);
    std::printf("host paths ok under the sanitizers (%d kernels registered)\n", n);
    return 0;
}
