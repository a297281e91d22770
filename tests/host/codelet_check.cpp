// CPU check of the register FFT codelets (turbofno_amd/csrc/fft_codelets.h compiled by the host compiler, with
// the vector types and function qualifiers supplied here): emulates the lanes of one L-lane group in a loop, performs the exchange as a
// plain matrix transpose, and compares the truncated forward / zero-padded backward transform of
// random data against a double-precision O(D^2) DFT. Prints "OK" and exits 0 on success.
#include <cmath>
struct float2 { float x, y; };
struct alignas(16) float4 { float x, y, z, w; };
static inline float2 make_float2(float x, float y) { return float2{ x, y }; }
#define TFNO_DEV static inline
#define TFNO_TABLE static const
#include "../../turbofno_amd/csrc/fft_codelets.h"
#include <complex>
#include <cstdio>
#include <cstdlib>
#include <vector>

using namespace tfno;
typedef std::complex<double> zd;

static double frand() { return 2.0 * rand() / RAND_MAX - 1.0; }

template <int LOGD> static double check_forward(bool use_table)
{
    constexpr int D = 1 << LOGD, L = D / 16;
    alignas(16) static cpx table[kTwLdsSize];
    for (int t = 0; t < L; ++t)
        for (int r = 0; r < 16; ++r) table[t * kTwLdsPitch + r] = kTwiddle1024[((t * r) << (10 - LOGD)) & 1023];
    std::vector<cpx> x(D);
    for (auto& v : x) v = make_float2((float)frand(), (float)frand());
    // pass 1 per lane
    std::vector<cpx> G(L * 16);
    for (int t = 0; t < L; ++t) {
        cpx v[16], tw[16], g[16];
        for (int i = 0; i < 16; ++i) v[i] = x[t + L * i];
        load_lane_twiddles<LOGD>(t, tw);
        if (use_table) {
            // the kernels' variant: twiddles from a pitch-18 table, transform split after the first radix-4 stage
            cpx bb[16];
            fft16_stage1<-1>(v, bb);
            fwd_pass1_lds_finish(bb, table + t * kTwLdsPitch, g);
        } else {
            fwd_pass1(v, tw, g);
        }
        for (int r = 0; r < 16; ++r) G[t * 16 + r] = g[r];
    }
    // pass 2 per output residue r
    std::vector<cpx> X(64);
    for (int r = 0; r < 16; ++r) {
        cpx out[4];
        if constexpr (L == 16) {
            cpx u[16];
            for (int t = 0; t < 16; ++t) u[t] = G[t * 16 + r];
            dft16_first4<-1>(u, out);
        } else {
            cpx u[8];
            for (int t = 0; t < 8; ++t) u[t] = G[t * 16 + r];
            dft8_first4<-1>(u, out);
        }
        for (int s = 0; s < 4; ++s) X[r + 16 * s] = out[s];
    }
    double num = 0, den = 0;
    for (int m = 0; m < 64; ++m) {
        zd acc = 0;
        for (int j = 0; j < D; ++j)
            acc += zd(x[j].x, x[j].y) * std::polar(1.0, -2.0 * M_PI * ((long)j * m % D) / D);
        num += std::norm(acc - zd(X[m].x, X[m].y));
        den += std::norm(acc);
    }
    return std::sqrt(num / den);
}

template <int LOGD> static double check_backward(bool use_table)
{
    constexpr int D = 1 << LOGD, L = D / 16;
    alignas(16) static cpx table[kTwLdsSize];
    for (int t = 0; t < L; ++t)
        for (int r = 0; r < 16; ++r) table[t * kTwLdsPitch + r] = kTwiddle1024[((t * r) << (10 - LOGD)) & 1023];
    std::vector<cpx> C(64);
    for (auto& v : C) v = make_float2((float)frand(), (float)frand());
    std::vector<cpx> H(16 * L);  // H[r][t]
    for (int r = 0; r < 16; ++r) {
        cpx c[4];
        for (int s = 0; s < 4; ++s) c[s] = C[r + 16 * s];
        if constexpr (L == 16) {
            cpx h[16];
            dft16_pad4<+1>(c, h);
            for (int t = 0; t < 16; ++t) H[r * L + t] = h[t];
        } else {
            cpx h[8];
            dft8_pad4<+1>(c, h);
            for (int t = 0; t < 8; ++t) H[r * L + t] = h[t];
        }
    }
    std::vector<cpx> y(D);
    for (int t = 0; t < L; ++t) {
        cpx e[16], tw[16], out[16];
        for (int r = 0; r < 16; ++r) e[r] = H[r * L + t];
        load_lane_twiddles<LOGD>(t, tw);
        if (use_table) inv_pass2_lds(e, table + t * kTwLdsPitch, out);
        else inv_pass2(e, tw, out);
        for (int i = 0; i < 16; ++i) y[t + L * i] = out[i];
    }
    double num = 0, den = 0;
    for (int j = 0; j < D; ++j) {
        zd acc = 0;
        for (int m = 0; m < 64; ++m)
            acc += zd(C[m].x, C[m].y) * std::polar(1.0, 2.0 * M_PI * ((long)j * m % D) / D);
        num += std::norm(acc - zd(y[j].x, y[j].y));
        den += std::norm(acc);
    }
    return std::sqrt(num / den);
}

// lengths 512 / 1024: lanes emulated in a loop around the same exchange array the kernels use
template <int LOGD> static double check_wide(bool backward)
{
    constexpr int D = 1 << LOGD, L = D / 16;
    std::vector<cpx> exch(L * 17);
    double num = 0, den = 0;
    if (!backward) {
        std::vector<cpx> x(D);
        for (auto& v : x) v = make_float2((float)frand(), (float)frand());
        for (int t = 0; t < L; ++t) {
            cpx v[16], tw[16], g[16];
            for (int i = 0; i < 16; ++i) v[i] = x[t + L * i];
            load_lane_twiddles<LOGD>(t, tw);
            fwd_pass1(v, tw, g);
            for (int r = 0; r < 16; ++r) exch[t * 17 + r] = g[r];
        }
        // second pass as the kernels run it: every lane's pruned 16-point transform, the small swap, the outer sums
        std::vector<cpx> swap(64 * (L / 16));
        for (int l = 0; l < L; ++l) {
            cpx inner[4];
            wide_forward_inner<L>(exch.data(), 1, l, inner);
            for (int c = 0; c < 4; ++c) swap[wide_swap_index<L>(l / (L / 16), c, l % (L / 16))] = inner[c];
        }
        std::vector<int> seen(64, 0);
        for (int l = 0; l < L; ++l) {
            cpx out[64 / L];
            wide_forward_outer<L>(swap.data(), 1, l, out);
            for (int j = 0; j < 64 / L; ++j) {
                const int m = wide_mode<L>(l, j);
                seen[m]++;
                const cpx X = out[j];
                zd acc = 0;
                for (int jj = 0; jj < D; ++jj) acc += zd(x[jj].x, x[jj].y) * std::polar(1.0, -2.0 * M_PI * ((long)jj * m % D) / D);
                num += std::norm(acc - zd(X.x, X.y));
                den += std::norm(acc);
            }
        }
        for (int m = 0; m < 64; ++m)
            if (seen[m] != 1) { printf("mode %d produced %d times\n", m, seen[m]); exit(1); }
    } else {
        for (int m = 0; m < 64; ++m) exch[m] = make_float2((float)frand(), (float)frand());
        std::vector<cpx> y(D);
        // first pass inputs as the kernels produce them: every lane's partial products, the second exchange, one row each
        std::vector<cpx> modes(exch.begin(), exch.begin() + 64), rows(L * 17);
        for (int l = 0; l < L; ++l) {
            cpx part[16];
            wide_backward_partial<L>(modes.data(), 1, l, part);
            for (int k = 0; k < 16; ++k) rows[wide_back_index<L>(l, k)] = part[k];
        }
        for (int t = 0; t < L; ++t) {
            cpx e[16], tw[16], out[16];
            for (int r = 0; r < 16; ++r) e[r] = rows[t * 17 + r];
            load_lane_twiddles<LOGD>(t, tw);
            inv_pass2(e, tw, out);
            for (int i = 0; i < 16; ++i) y[t + L * i] = out[i];
        }
        for (int j = 0; j < D; ++j) {
            zd acc = 0;
            for (int m = 0; m < 64; ++m) acc += zd(exch[m].x, exch[m].y) * std::polar(1.0, 2.0 * M_PI * ((long)j * m % D) / D);
            num += std::norm(acc - zd(y[j].x, y[j].y));
            den += std::norm(acc);
        }
    }
    return std::sqrt(num / den);
}

// rows of 128 handled by 16 lanes, two rows of 8 samples per lane (the whole-image kernels' row pass for DY = 128):
// lane t holds samples t + 16 i of row A and row B, after the exchange lane t = r + 8 h finishes row h, modes r + 8 c.
static double check_rows128(bool backward)
{
    constexpr int D = 128;
    std::vector<cpx> exch(16 * 17);
    cpx tw[16][8];
    for (int t = 0; t < 16; ++t)
        for (int r = 0; r < 8; ++r) tw[t][r] = kTwiddle1024[((t * r) << 3) & 1023];
    double num = 0, den = 0;
    if (!backward) {
        std::vector<cpx> x(2 * D);
        for (auto& v : x) v = make_float2((float)frand(), (float)frand());
        for (int t = 0; t < 16; ++t) {
            cpx a[8], b[8];
            for (int i = 0; i < 8; ++i) { a[i] = x[t + 16 * i]; b[i] = x[D + t + 16 * i]; }
            fft8<-1>(a);
            fft8<-1>(b);
            for (int r = 0; r < 8; ++r) { exch[t * 17 + r] = cmul(a[r], tw[t][r]); exch[t * 17 + 8 + r] = cmul(b[r], tw[t][r]); }
        }
        for (int t = 0; t < 16; ++t) {
            cpx u[16], out[8];
            for (int tt = 0; tt < 16; ++tt) u[tt] = exch[tt * 17 + t];
            dft16_first8<-1>(u, out);
            const int row = t >> 3, r = t & 7;
            for (int c = 0; c < 8; ++c) {
                const int m = r + 8 * c;
                zd acc = 0;
                for (int j = 0; j < D; ++j)
                    acc += zd(x[row * D + j].x, x[row * D + j].y) * std::polar(1.0, -2.0 * M_PI * ((long)j * m % D) / D);
                num += std::norm(acc - zd(out[c].x, out[c].y));
                den += std::norm(acc);
            }
        }
    } else {
        std::vector<cpx> C(2 * 64), y(2 * D);
        for (auto& v : C) v = make_float2((float)frand(), (float)frand());
        for (int t = 0; t < 16; ++t) {
            const int row = t >> 3, r = t & 7;
            cpx c[8], h[16];
            for (int k = 0; k < 8; ++k) c[k] = C[row * 64 + r + 8 * k];
            dft16_pad8<+1>(c, h);
            for (int tt = 0; tt < 16; ++tt) exch[tt * 17 + t] = h[tt];
        }
        for (int t = 0; t < 16; ++t) {
            cpx a[8], b[8];
            for (int r = 0; r < 8; ++r) { a[r] = cmulc(exch[t * 17 + r], tw[t][r]); b[r] = cmulc(exch[t * 17 + 8 + r], tw[t][r]); }
            fft8<+1>(a);
            fft8<+1>(b);
            for (int i = 0; i < 8; ++i) { y[t + 16 * i] = a[i]; y[D + t + 16 * i] = b[i]; }
        }
        for (int row = 0; row < 2; ++row)
            for (int j = 0; j < D; ++j) {
                zd acc = 0;
                for (int m = 0; m < 64; ++m)
                    acc += zd(C[row * 64 + m].x, C[row * 64 + m].y) * std::polar(1.0, 2.0 * M_PI * ((long)j * m % D) / D);
                num += std::norm(acc - zd(y[row * D + j].x, y[row * D + j].y));
                den += std::norm(acc);
            }
    }
    return std::sqrt(num / den);
}

int main()
{
    srand(12345);
    double e[8] = { check_forward<8>(false), check_forward<7>(false), check_backward<8>(false), check_backward<7>(false),
                    check_forward<8>(true),  check_forward<7>(true),  check_backward<8>(true),  check_backward<7>(true) };
    printf("registers: fwd256 %.3e fwd128 %.3e bwd256 %.3e bwd128 %.3e\n", e[0], e[1], e[2], e[3]);
    printf("table    : fwd256 %.3e fwd128 %.3e bwd256 %.3e bwd128 %.3e\n", e[4], e[5], e[6], e[7]);
    double w[4] = { check_wide<9>(false), check_wide<10>(false), check_wide<9>(true), check_wide<10>(true) };
    printf("wide     : fwd512 %.3e fwd1024 %.3e bwd512 %.3e bwd1024 %.3e\n", w[0], w[1], w[2], w[3]);
    for (double v : e)
        if (!(v < 5e-7)) { printf("FAIL\n"); return 1; }
    for (double v : w)
        if (!(v < 5e-7)) { printf("FAIL\n"); return 1; }
    const double p0 = check_rows128(false), p1 = check_rows128(true);
    printf("rows128  : fwd %.3e bwd %.3e\n", p0, p1);
    if (!(p0 < 5e-7) || !(p1 < 5e-7)) { printf("FAIL\n"); return 1; }
    printf("OK\n");
    return 0;
}
