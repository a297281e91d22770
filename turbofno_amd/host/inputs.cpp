#include "inputs.h"
#include <cmath>
#include <complex>
#include <cstring>
#include <random>

namespace {

typedef std::complex<double> zd;

// in-place radix-2 transform of n = 2^p values with stride `stride`; sign = +1: exp(+2 pi i jk/n), unnormalised
void fft_inplace(zd* a, int n, long stride, int sign)
{
    for (int i = 1, j = 0; i < n; ++i) {
        int bit = n >> 1;
        for (; j & bit; bit >>= 1) j ^= bit;
        j ^= bit;
        if (i < j) std::swap(a[i * stride], a[j * stride]);
    }
    for (int len = 2; len <= n; len <<= 1) {
        const double ang = sign * 2.0 * M_PI / len;
        const zd wl(std::cos(ang), std::sin(ang));
        for (int i = 0; i < n; i += len) {
            zd w(1.0, 0.0);
            for (int j = 0; j < len / 2; ++j) {
                const zd u = a[(i + j) * stride], v = a[(i + j + len / 2) * stride] * w;
                a[(i + j) * stride] = u + v;
                a[(i + j + len / 2) * stride] = u - v;
                w *= wl;
            }
        }
    }
}

}  // namespace

InputKind input_kind_from_name(const char* name)
{
    if (!name) return InputKind::reference_rand;
    if (!strcmp(name, "uniform")) return InputKind::uniform;
    if (!strcmp(name, "smooth")) return InputKind::smooth;
    if (!strcmp(name, "vorticity")) return InputKind::vorticity;
    return InputKind::reference_rand;
}

uint64_t default_seed(InputKind kind)
{
    switch (kind) {
    case InputKind::uniform: return 0x5EED + 2;
    case InputKind::smooth: return 0x5EED + 3;
    case InputKind::vorticity: return 0x5EED + 5;
    default: return 0x5EED;
    }
}

std::vector<float> generate_inputs(InputKind kind, uint64_t seed, int channels, long signals, int dx, int dy)
{
    const size_t total = (size_t)channels * signals * dy;
    std::vector<float> out(2 * total);
    std::mt19937_64 rng(seed);
    if (kind == InputKind::uniform || kind == InputKind::reference_rand) {
        std::uniform_real_distribution<float> u(-1.0f, 1.0f);
        for (auto& v : out) v = u(rng);
    } else if (kind == InputKind::smooth) {
        std::uniform_int_distribution<int> freq(1, 32);
        std::uniform_real_distribution<double> phase(0.0, 2.0 * M_PI);
        std::normal_distribution<double> noise(0.0, 1.0);
        for (size_t sig = 0; sig < (size_t)channels * signals; ++sig)
            for (int part = 0; part < 2; ++part) {          // real part, then an independent imaginary part
                int f[8];
                double ph[8];
                for (int i = 0; i < 8; ++i) { f[i] = freq(rng); ph[i] = phase(rng); }
                for (int j = 0; j < dy; ++j) {
                    double v = 0.01 * noise(rng);
                    for (int i = 0; i < 8; ++i) v += std::sin(2.0 * M_PI * f[i] * j / dy + ph[i]);
                    out[2 * (sig * dy + j) + part] = (float)v;
                }
            }
    } else {
        // vorticity: one DX x DY field per (channel, batch element); signals = bs * DX
        const int DX = dx > 0 ? dx : 1;
        const long bs = signals / DX;
        std::normal_distribution<double> normal(0.0, 1.0);
        std::vector<zd> field((size_t)DX * dy);
        for (int k = 0; k < channels; ++k) {
            const size_t chan0 = (size_t)k * signals * dy;
            double power = 0.0;
            for (long b = 0; b < bs; ++b) {
                for (int p = 0; p < DX; ++p)
                    for (int q = 0; q < dy; ++q) {
                        const double kx = p <= DX / 2 - (DX % 2 == 0) ? p : p - DX;    // numpy.fft.fftfreq ordering (Nyquist negative)
                        const double ky = q <= dy / 2 - (dy % 2 == 0) ? q : q - dy;
                        const double amp = std::pow(kx * kx + ky * ky + 9.0, -1.25);
                        field[(size_t)p * dy + q] = zd(normal(rng), normal(rng)) * amp;
                    }
                for (int p = 0; p < DX; ++p) fft_inplace(&field[(size_t)p * dy], dy, 1, +1);
                for (int q = 0; q < dy; ++q) fft_inplace(&field[q], DX, dy, +1);
                for (size_t i = 0; i < field.size(); ++i) {
                    power += std::norm(field[i]);
                    out[2 * (chan0 + (size_t)b * DX * dy + i)] = (float)field[i].real();
                    out[2 * (chan0 + (size_t)b * DX * dy + i) + 1] = (float)field[i].imag();
                }
            }
            // unit variance per channel (the fields have zero mean by construction of the spectrum's phases)
            const float scale = (float)(1.0 / std::sqrt(power / ((double)signals * dy)));
            for (size_t i = 0; i < (size_t)signals * dy; ++i) {
                out[2 * (chan0 + i)] *= scale;
                out[2 * (chan0 + i) + 1] *= scale;
            }
        }
    }
    return out;
}

std::vector<float> generate_weights(InputKind kind, uint64_t seed, int K, int N)
{
    std::vector<float> w(2 * (size_t)K * N);
    std::mt19937_64 rng(seed ^ 0x9E3779B97F4A7C15ull);      // a stream of its own, independent of the input's
    const float s = 1.0f / std::sqrt((float)K);
    if (kind == InputKind::vorticity) {
        std::normal_distribution<float> n(0.0f, 1.0f);
        for (auto& v : w) v = n(rng) * s;
    } else {
        std::uniform_real_distribution<float> u(-1.0f, 1.0f);
        for (auto& v : w) v = u(rng) * s;
    }
    return w;
}
