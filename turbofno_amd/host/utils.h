// Host-side helpers of the drivers: config-file grammar, random fill, HIP error checks.
// Counterparts in the reference: utils/utils.cu:14-22 (parse_line), :37-43 (generate_random_vector),
// utils/utils.cuh:17-25 (kernel check that exits), :43-57 (runtime-call check that only prints).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdio>
#include <algorithm>
#include <cstdlib>
#include <map>
#include <string>
#include <vector>

// values of one "key = v v v" line (the first two tokens are skipped)
std::vector<int> parse_line(const std::string& line);

// whole file -> key -> values; '#' comments and blank lines are skipped; a missing file yields an
// empty map (the reference's unchecked ifstream behaves the same: zero problems are run)
std::map<std::string, std::vector<int>> load_problem_config(const std::string& path);

// +-{0..9} * 1e-3 from rand(), unseeded: the reference's input distribution
void generate_random_vector(float* target, long n);

// Inputs of one problem in two steps, so that the draws from rand() can precede every HIP call of the problem (the HIP
// runtime's own threads draw from rand() once it is initialised, which would make the values depend on timing):
//   draw_random(n)          min(n, 2^22) values of generate_random_vector's distribution, exactly as the reference's mains
//                           draw them (utils/utils.cu:37-43, fused.cu:61-62);
//   upload_tiled(dev, n, v) fills a device buffer of n floats with v, repeated (device-to-device copies) when n is larger:
//                           drawing gigabytes from rand() per problem takes longer than the whole sweep, and the reference
//                           fills its one fixed-size buffer once per process instead (fused.cu:25-45,61).
std::vector<float> draw_random(size_t n);
void upload_tiled(void* device, size_t n, const std::vector<float>& values);

// With TURBOFNO_DIGEST set in the environment the drivers print, after the warm-up launch of each problem, one
// line "digest: <weighted sum re> <weighted sum im> <sum |y|^2>" of the output on stderr, and reseed rand() before
// generating each problem's inputs: every variant of a problem then sees the same inputs and must print the same
// digest up to fp32 rounding.
void print_output_digest(const void* device_y, size_t complex_elems);

// With TURBOFNO_STATS set the drivers add, after the reference-format result line, one line
// "  stats: min=<ms> median=<ms> max=<ms> over <n> iterations" from per-iteration events around the same launches
// (the result line itself stays the mean over launch + device synchronise, as in the reference).
template <class Launch> void print_iteration_stats(Launch&& launch, int n)
{
    std::vector<hipEvent_t> ev(2 * (size_t)n);
    for (auto& e : ev) (void)hipEventCreate(&e);
    for (int i = 0; i < n; ++i) {
        (void)hipEventRecord(ev[2 * i]);
        launch();
        (void)hipEventRecord(ev[2 * i + 1]);
        (void)hipDeviceSynchronize();
    }
    std::vector<float> ms(n);
    for (int i = 0; i < n; ++i) (void)hipEventElapsedTime(&ms[i], ev[2 * i], ev[2 * i + 1]);
    std::sort(ms.begin(), ms.end());
    printf("  stats: min=%.4fms median=%.4fms max=%.4fms over %d iterations\n", ms.front(), ms[n / 2], ms.back(), n);
    fflush(stdout);
    for (auto& e : ev) (void)hipEventDestroy(e);
}

#define HIP_RT_CALL(call)                                                                                    \
    do {                                                                                                     \
        hipError_t status_ = (call);                                                                         \
        if (status_ != hipSuccess)                                                                           \
            fprintf(stderr, "HIP runtime error at %s:%d: %s (%d)\n", __FILE__, __LINE__,                     \
                    hipGetErrorString(status_), (int)status_);                                               \
    } while (0)

#define CHECK_HIP_KERNEL()                                                                                   \
    do {                                                                                                     \
        hipError_t status_ = hipGetLastError();                                                              \
        if (status_ != hipSuccess) {                                                                         \
            fprintf(stderr, "kernel error at %s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(status_)); \
            exit(EXIT_FAILURE);                                                                              \
        }                                                                                                    \
    } while (0)

#define CHECK_TURBOFNO(call)                                                                                 \
    do {                                                                                                     \
        int rc_ = (call);                                                                                    \
        if (rc_ != 0) {                                                                                      \
            fprintf(stderr, "turbofno error %d at %s:%d: %s\n", rc_, __FILE__, __LINE__,                     \
                    turbofno_last_error_string());                                                           \
            exit(EXIT_FAILURE);                                                                              \
        }                                                                                                    \
    } while (0)
