// CPU check of the group transforms of turbofno_amd/csrc/group_fft.h AS THE KERNELS RUN THEM: every lane of an L-lane
// group is a host thread that executes the device function of that lane, the exchange array is shared, and
// wave_lds_fence() is a barrier over the L threads (on the GPU the lanes of a wavefront run in lockstep). This covers
// what the loop emulation in codelet_check.cpp cannot: the layouts of the exchanges (who writes where, who reads what)
// of lengths 128 to 1024, with twiddle powers from the table and from an array. Compared against a double-precision
// O(D^2) DFT of the 64 retained modes. Prints "OK" and exits 0 on success.
#include <cmath>
struct float2 { float x, y; };
struct alignas(16) float4 { float x, y, z, w; };
static inline float2 make_float2(float x, float y) { return float2{ x, y }; }
#define TFNO_DEV static inline
#define TFNO_TABLE static const
#include "../../turbofno_amd/csrc/group_fft.h"
#include <complex>
#include <cstdio>
#include <cstdlib>
#include <pthread.h>
#include <thread>
#include <vector>

static pthread_barrier_t g_lanes;
namespace tfno {
void wave_lds_fence() { pthread_barrier_wait(&g_lanes); }
}
using namespace tfno;
typedef std::complex<double> zd;
static double frand() { return 2.0 * rand() / RAND_MAX - 1.0; }

template <class F> static void run_lanes(int L, F lane)
{
    pthread_barrier_init(&g_lanes, nullptr, (unsigned)L);
    std::vector<std::thread> th;
    for (int t = 0; t < L; ++t) th.emplace_back(lane, t);
    for (auto& x : th) x.join();
    pthread_barrier_destroy(&g_lanes);
}

// forward: samples in, 64 modes out through forward_mode_of_lane. pow_from_array: the variant of the whole-image kernels
template <int LOGD> static double check_forward(bool pow_from_array)
{
    constexpr int D = 1 << LOGD, L = D / 16, MM = 64 / L;
    std::vector<cpx> x(D), exch(L * 17 + 64), X(64), wsm(L);
    std::vector<int> seen(64, 0);
    for (auto& v : x) v = make_float2((float)frand(), (float)frand());
    for (int e = 0; e < L; ++e) wsm[e] = kTwiddle1024[e * (1024 / L)];
    run_lanes(L, [&](int t) {
        cpx v[16], tw[16], g[16], out[MM];
        for (int i = 0; i < 16; ++i) v[i] = x[t + L * i];
        load_lane_twiddles<LOGD>(t, tw);
        fwd_pass1(v, tw, g);
        if constexpr (L >= 32) {
            if (pow_from_array) wide_forward_finish<L, true>(g, exch.data(), wsm.data(), t, out);
            else group_forward_finish<LOGD>(g, exch.data(), t, out);
        } else {
            group_forward_finish<LOGD>(g, exch.data(), t, out);
        }
        for (int mm = 0; mm < MM; ++mm) {
            const int m = forward_mode_of_lane<LOGD>(t, mm);
            X[m] = out[mm];                       // distinct lanes write distinct modes (checked below)
            __atomic_fetch_add(&seen[m], 1, __ATOMIC_RELAXED);
        }
    });
    double num = 0, den = 0;
    for (int m = 0; m < 64; ++m) {
        if (seen[m] != 1) { printf("length %d: mode %d produced %d times\n", D, m, seen[m]); exit(1); }
        zd acc = 0;
        for (int j = 0; j < D; ++j) acc += zd(x[j].x, x[j].y) * std::polar(1.0, -2.0 * M_PI * ((long)j * m % D) / D);
        num += std::norm(acc - zd(X[m].x, X[m].y));
        den += std::norm(acc);
    }
    return std::sqrt(num / den);
}

// backward: 64 modes (lane t holds t + L mm) in, D samples out
template <int LOGD> static double check_backward(bool pow_from_array)
{
    constexpr int D = 1 << LOGD, L = D / 16, MM = 64 / L;
    std::vector<cpx> C(64), exch(L * 17 + 64), y(D), wsm(L);
    for (auto& v : C) v = make_float2((float)frand(), (float)frand());
    for (int e = 0; e < L; ++e) wsm[e] = kTwiddle1024[e * (1024 / L)];
    run_lanes(L, [&](int t) {
        cpx c[MM], tw[16], out[16];
        for (int mm = 0; mm < MM; ++mm) c[mm] = C[t + L * mm];
        load_lane_twiddles<LOGD>(t, tw);
        if constexpr (L >= 32) {
            if (pow_from_array) {
                cpx e[16];
                wide_backward_inputs<L, true>(c, wsm.data(), exch.data(), t, e);
                inv_pass2(e, tw, out);
            } else {
                group_backward<LOGD>(c, tw, exch.data(), t, out);
            }
        } else {
            group_backward<LOGD>(c, tw, exch.data(), t, out);
        }
        for (int i = 0; i < 16; ++i) y[t + L * i] = out[i];
    });
    double num = 0, den = 0;
    for (int j = 0; j < D; ++j) {
        zd acc = 0;
        for (int m = 0; m < 64; ++m) acc += zd(C[m].x, C[m].y) * std::polar(1.0, 2.0 * M_PI * ((long)j * m % D) / D);
        num += std::norm(acc - zd(y[j].x, y[j].y));
        den += std::norm(acc);
    }
    return std::sqrt(num / den);
}

int main()
{
    srand(4321);
    const double f[6] = { check_forward<7>(false), check_forward<8>(false), check_forward<9>(false), check_forward<10>(false),
                          check_forward<9>(true),  check_forward<10>(true) };
    const double b[6] = { check_backward<7>(false), check_backward<8>(false), check_backward<9>(false), check_backward<10>(false),
                          check_backward<9>(true),  check_backward<10>(true) };
    printf("forward : 128 %.3e 256 %.3e 512 %.3e 1024 %.3e | powers from an array: 512 %.3e 1024 %.3e\n", f[0], f[1], f[2], f[3], f[4], f[5]);
    printf("backward: 128 %.3e 256 %.3e 512 %.3e 1024 %.3e | powers from an array: 512 %.3e 1024 %.3e\n", b[0], b[1], b[2], b[3], b[4], b[5]);
    for (double v : f)
        if (!(v < 5e-7)) { printf("FAIL\n"); return 1; }
    for (double v : b)
        if (!(v < 5e-7)) { printf("FAIL\n"); return 1; }
    printf("OK\n");
    return 0;
}
