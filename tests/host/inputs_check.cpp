// CPU check of the drivers' seeded input generators (turbofno_amd/host/inputs.cpp): prints one line of statistics per
// kind, "kind min max mean var lowband" where lowband = share of a signal's energy in bins |f| <= 32, so that the
// Python test can check ranges, unit variance, smoothness and that (kind, seed) is reproducible.
#include "../../turbofno_amd/host/inputs.h"
#include <cmath>
#include <complex>
#include <cstdio>
#include <cstdlib>

static void stats(const char* name, const std::vector<float>& v, int dy)
{
    double mn = 1e30, mx = -1e30, s = 0, s2 = 0;
    for (float f : v) { mn = f < mn ? f : mn; mx = f > mx ? f : mx; s += f; s2 += (double)f * f; }
    const size_t n = v.size();
    // energy share of the low band in the first signal (brute-force DFT)
    double low = 0, all = 0;
    for (int m = 0; m < dy; ++m) {
        std::complex<double> acc = 0;
        for (int j = 0; j < dy; ++j) acc += std::complex<double>(v[2 * j], v[2 * j + 1]) * std::polar(1.0, -2.0 * M_PI * j * m / dy);
        const int f = m <= dy / 2 ? m : dy - m;
        all += std::norm(acc);
        if (f <= 32) low += std::norm(acc);
    }
    printf("%s %.6f %.6f %.6f %.6f %.6f\n", name, mn, mx, s / n, 2.0 * (s2 / n), low / all);   // var of the complex values = 2 * mean square of the floats
}

int main()
{
    const int K = 4, dy = 128;
    stats("uniform", generate_inputs(InputKind::uniform, 7, K, 6, 0, dy), dy);
    stats("smooth", generate_inputs(InputKind::smooth, 7, K, 6, 0, dy), dy);
    stats("vorticity", generate_inputs(InputKind::vorticity, 7, K, 2 * 64, 64, dy), dy);
    const auto a = generate_inputs(InputKind::smooth, 11, 2, 3, 0, dy), b = generate_inputs(InputKind::smooth, 11, 2, 3, 0, dy),
               c = generate_inputs(InputKind::smooth, 12, 2, 3, 0, dy);
    printf("reproducible %d\ndiffers %d\n", (int)(a == b), (int)(a != c));
    const auto wu = generate_weights(InputKind::uniform, 7, 16, 64), wn = generate_weights(InputKind::vorticity, 7, 16, 64);
    double mxu = 0, s2n = 0;
    for (float f : wu) mxu = std::fabs(f) > mxu ? std::fabs(f) : mxu;
    for (float f : wn) s2n += (double)f * f;
    printf("weights %.6f %.6f\n", mxu, 2.0 * s2n / wn.size() * 16);    // max |uniform| <= 1/sqrt(K); K * var(normal) = 2
    return 0;
}
