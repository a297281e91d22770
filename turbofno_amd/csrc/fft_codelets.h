// Register-resident FFT building blocks for 64-lane wavefronts (gfx950).
//
// These replace the reference's auto-generated radix-2 codelets, whose sources live in the empty
// TurboFFT submodule (include sites: fusion_variants/1D_D_exp_fused_fft_cgemm_ifft/
// fused_fft_cgemm_ifft_7.cuh:3-4, call sites :46,114,218). A length-D transform (D = 16*L) is split as
//
//     y = t + L*i            t < L : lane inside an L-lane group,  i < 16 : register index
//     G_t[r]   = sum_i v[t + L*i] w16^(i r)                      16-point FFT, all in registers
//     X[r+16s] = sum_t w_D^(t r) w_L^(t s) G_t[r]                one exchange, then an L-point DFT
//
// Truncation to 64 modes means only s < 4 is ever needed ("pruned" second pass: 16 in, 4 out);
// the zero-padded backward transform is the exact mirror (4 in, 16 out, exchange, 16-point FFT).
// Discarded and padded modes are therefore never computed, stored or loaded.
//
// DIR = -1 is the forward transform exp(-2 pi i jm/D); DIR = +1 the unnormalised backward one.
#pragma once
// The arithmetic below is plain C++ over float2 / float4: a translation unit that is not compiled by hipcc (a CPU
// unit test of the codelets) defines TFNO_DEV, TFNO_TABLE and those two vector types before including this header.
#ifndef TFNO_DEV
#include <hip/hip_runtime.h>
#define TFNO_DEV __device__ __forceinline__
#define TFNO_TABLE __device__ __constant__ const
#endif

namespace tfno {

using cpx = float2;

TFNO_TABLE float2 kTwiddle1024[1024] = {
#include "twiddles_1024.inc"
};

TFNO_DEV cpx cadd(cpx a, cpx b) { return make_float2(a.x + b.x, a.y + b.y); }
TFNO_DEV cpx csub(cpx a, cpx b) { return make_float2(a.x - b.x, a.y - b.y); }
TFNO_DEV cpx cmul(cpx a, cpx b) { return make_float2(a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x); }
TFNO_DEV cpx cmulc(cpx a, cpx b) { return make_float2(a.x * b.x + a.y * b.y, a.y * b.x - a.x * b.y); }  // a * conj(b)
TFNO_DEV void cfma(cpx& acc, cpx a, cpx b)
{
    acc.x = fmaf(a.x, b.x, acc.x); acc.x = fmaf(-a.y, b.y, acc.x);
    acc.y = fmaf(a.x, b.y, acc.y); acc.y = fmaf(a.y, b.x, acc.y);
}

// multiply by DIR * i   (forward: -i, backward: +i)
template <int DIR> TFNO_DEV cpx mul_dir_i(cpx a)
{
    return DIR < 0 ? make_float2(a.y, -a.x) : make_float2(-a.y, a.x);
}

// w16^k for the forward direction, k = 0..15 (compile-time constants)
template <int K16> TFNO_DEV constexpr float w16_re()
{
    constexpr float c[16] = { 1.0f, 0.92387953251128674f, 0.70710678118654752f, 0.38268343236508977f,
                              0.0f, -0.38268343236508977f, -0.70710678118654752f, -0.92387953251128674f,
                              -1.0f, -0.92387953251128674f, -0.70710678118654752f, -0.38268343236508977f,
                              0.0f, 0.38268343236508977f, 0.70710678118654752f, 0.92387953251128674f };
    return c[K16 & 15];
}
template <int K16> TFNO_DEV constexpr float w16_im()
{
    constexpr float s[16] = { 0.0f, -0.38268343236508977f, -0.70710678118654752f, -0.92387953251128674f,
                              -1.0f, -0.92387953251128674f, -0.70710678118654752f, -0.38268343236508977f,
                              0.0f, 0.38268343236508977f, 0.70710678118654752f, 0.92387953251128674f,
                              1.0f, 0.92387953251128674f, 0.70710678118654752f, 0.38268343236508977f };
    return s[K16 & 15];
}

// a * w16^(DIR-signed k)
template <int DIR, int K16> TFNO_DEV cpx mul_w16(cpx a)
{
    constexpr int k = K16 & 15;
    if constexpr (k == 0) return a;
    else if constexpr (k == 4) return mul_dir_i<DIR>(a);
    else if constexpr (k == 8) return make_float2(-a.x, -a.y);
    else if constexpr (k == 12) return mul_dir_i<-DIR>(a);
    else {
        constexpr float wr = w16_re<k>();
        constexpr float wi = DIR < 0 ? w16_im<k>() : -w16_im<k>();
        return make_float2(a.x * wr - a.y * wi, a.x * wi + a.y * wr);
    }
}

// 4-point butterfly, in place, natural order out
template <int DIR> TFNO_DEV void radix4(cpx& a0, cpx& a1, cpx& a2, cpx& a3)
{
    cpx t0 = cadd(a0, a2), t1 = csub(a0, a2), t2 = cadd(a1, a3), t3 = mul_dir_i<DIR>(csub(a1, a3));
    a0 = cadd(t0, t2); a1 = cadd(t1, t3); a2 = csub(t0, t2); a3 = csub(t1, t3);
}

// position of output bin r inside the array after fft16(): X[r] = v[fft16_slot(r)]
TFNO_DEV constexpr int fft16_slot(int r) { return (r >> 2) | ((r & 3) << 2); }

// 16-point FFT in registers. Input natural order v[i]; output bin r is left in v[fft16_slot(r)].
template <int DIR> TFNO_DEV void fft16(cpx (&v)[16])
{
#pragma unroll
    for (int i0 = 0; i0 < 4; ++i0) radix4<DIR>(v[i0], v[i0 + 4], v[i0 + 8], v[i0 + 12]);
    // v[i0 + 4 rho] = B[i0][rho]; twiddle by w16^(i0*rho)
    v[5] = mul_w16<DIR, 1>(v[5]);   v[9] = mul_w16<DIR, 2>(v[9]);   v[13] = mul_w16<DIR, 3>(v[13]);
    v[6] = mul_w16<DIR, 2>(v[6]);   v[10] = mul_w16<DIR, 4>(v[10]); v[14] = mul_w16<DIR, 6>(v[14]);
    v[7] = mul_w16<DIR, 3>(v[7]);   v[11] = mul_w16<DIR, 6>(v[11]); v[15] = mul_w16<DIR, 9>(v[15]);
#pragma unroll
    for (int rho = 0; rho < 4; ++rho) radix4<DIR>(v[4 * rho], v[4 * rho + 1], v[4 * rho + 2], v[4 * rho + 3]);
}

// The same transform in two steps, out of place: fft16_stage1 reads v[] and leaves the first radix-4
// stage (twiddled) in b[]; after it v[] is dead, so the caller can reuse those registers (e.g. as the
// landing zone of the next row's loads) while fft16_stage2 finishes in b[].
template <int DIR> TFNO_DEV void fft16_stage1(const cpx (&v)[16], cpx (&b)[16])
{
#pragma unroll
    for (int i0 = 0; i0 < 4; ++i0) {
        cpx a0 = v[i0], a1 = v[i0 + 4], a2 = v[i0 + 8], a3 = v[i0 + 12];
        radix4<DIR>(a0, a1, a2, a3);
        b[i0] = a0; b[i0 + 4] = a1; b[i0 + 8] = a2; b[i0 + 12] = a3;
    }
    b[5] = mul_w16<DIR, 1>(b[5]);   b[9] = mul_w16<DIR, 2>(b[9]);   b[13] = mul_w16<DIR, 3>(b[13]);
    b[6] = mul_w16<DIR, 2>(b[6]);   b[10] = mul_w16<DIR, 4>(b[10]); b[14] = mul_w16<DIR, 6>(b[14]);
    b[7] = mul_w16<DIR, 3>(b[7]);   b[11] = mul_w16<DIR, 6>(b[11]); b[15] = mul_w16<DIR, 9>(b[15]);
}
template <int DIR> TFNO_DEV void fft16_stage2(cpx (&b)[16])
{
#pragma unroll
    for (int rho = 0; rho < 4; ++rho) radix4<DIR>(b[4 * rho], b[4 * rho + 1], b[4 * rho + 2], b[4 * rho + 3]);
}

// First four bins (s = 0..3) of a 16-point DFT of g[0..15]:  out[s] = sum_t g[t] w16^(t s).
template <int DIR> TFNO_DEV void dft16_first4(cpx (&g)[16], cpx (&out)[4])
{
#pragma unroll
    for (int t0 = 0; t0 < 4; ++t0) radix4<DIR>(g[t0], g[t0 + 4], g[t0 + 8], g[t0 + 12]);
    // g[t0 + 4 s] = sum_t1 g[t0 + 4 t1] w4^(t1 s);  out[s] = sum_t0 w16^(t0 s) g[t0 + 4 s]
    out[0] = cadd(cadd(g[0], g[1]), cadd(g[2], g[3]));
    out[1] = cadd(cadd(g[4], mul_w16<DIR, 1>(g[5])), cadd(mul_w16<DIR, 2>(g[6]), mul_w16<DIR, 3>(g[7])));
    out[2] = cadd(cadd(g[8], mul_w16<DIR, 2>(g[9])), cadd(mul_w16<DIR, 4>(g[10]), mul_w16<DIR, 6>(g[11])));
    out[3] = cadd(cadd(g[12], mul_w16<DIR, 3>(g[13])), cadd(mul_w16<DIR, 6>(g[14]), mul_w16<DIR, 9>(g[15])));
}

// 16-point DFT of a 4-element input padded with 12 zeros:  h[t] = sum_{s<4} c[s] w16^(t s), t = 0..15.
template <int DIR> TFNO_DEV void dft16_pad4(const cpx (&c)[4], cpx (&h)[16])
{
    // t = t0 + 4 t1:  h[t0 + 4 t1] = sum_s (c[s] w16^(t0 s)) w4^(t1 s)
    {
        cpx d0 = c[0], d1 = c[1], d2 = c[2], d3 = c[3];
        radix4<DIR>(d0, d1, d2, d3); h[0] = d0; h[4] = d1; h[8] = d2; h[12] = d3;
    }
    {
        cpx d0 = c[0], d1 = mul_w16<DIR, 1>(c[1]), d2 = mul_w16<DIR, 2>(c[2]), d3 = mul_w16<DIR, 3>(c[3]);
        radix4<DIR>(d0, d1, d2, d3); h[1] = d0; h[5] = d1; h[9] = d2; h[13] = d3;
    }
    {
        cpx d0 = c[0], d1 = mul_w16<DIR, 2>(c[1]), d2 = mul_w16<DIR, 4>(c[2]), d3 = mul_w16<DIR, 6>(c[3]);
        radix4<DIR>(d0, d1, d2, d3); h[2] = d0; h[6] = d1; h[10] = d2; h[14] = d3;
    }
    {
        cpx d0 = c[0], d1 = mul_w16<DIR, 3>(c[1]), d2 = mul_w16<DIR, 6>(c[2]), d3 = mul_w16<DIR, 9>(c[3]);
        radix4<DIR>(d0, d1, d2, d3); h[3] = d0; h[7] = d1; h[11] = d2; h[15] = d3;
    }
}

// First four bins of an 8-point DFT:  out[s] = sum_{t<8} g[t] w8^(t s), s = 0..3.
template <int DIR> TFNO_DEV void dft8_first4(cpx (&g)[8], cpx (&out)[4])
{
    // t = t0 + 2 t1:  B[t0][s] = sum_t1 g[t0 + 2 t1] w4^(t1 s);  out[s] = B[0][s] + w8^s B[1][s]
    radix4<DIR>(g[0], g[2], g[4], g[6]);
    radix4<DIR>(g[1], g[3], g[5], g[7]);
    out[0] = cadd(g[0], g[1]);
    out[1] = cadd(g[2], mul_w16<DIR, 2>(g[3]));
    out[2] = cadd(g[4], mul_w16<DIR, 4>(g[5]));
    out[3] = cadd(g[6], mul_w16<DIR, 6>(g[7]));
}

// 8-point DFT of a 4-element input padded with 4 zeros:  h[t] = sum_{s<4} c[s] w8^(t s), t = 0..7.
template <int DIR> TFNO_DEV void dft8_pad4(const cpx (&c)[4], cpx (&h)[8])
{
    {
        cpx d0 = c[0], d1 = c[1], d2 = c[2], d3 = c[3];
        radix4<DIR>(d0, d1, d2, d3); h[0] = d0; h[2] = d1; h[4] = d2; h[6] = d3;
    }
    {
        cpx d0 = c[0], d1 = mul_w16<DIR, 2>(c[1]), d2 = mul_w16<DIR, 4>(c[2]), d3 = mul_w16<DIR, 6>(c[3]);
        radix4<DIR>(d0, d1, d2, d3); h[1] = d0; h[3] = d1; h[5] = d2; h[7] = d3;
    }
}

// 8-point FFT in registers, natural order in and out.
template <int DIR> TFNO_DEV void fft8(cpx (&v)[8])
{
    // i = i0 + 2 i1:  B_i0[rho] = sum_i1 v[i0 + 2 i1] w4^(i1 rho);  F[rho + 4 sigma] = B_0[rho] + (-1)^sigma w8^rho B_1[rho]
    radix4<DIR>(v[0], v[2], v[4], v[6]);
    radix4<DIR>(v[1], v[3], v[5], v[7]);
    const cpx w0 = v[1], w1 = mul_w16<DIR, 2>(v[3]), w2 = mul_w16<DIR, 4>(v[5]), w3 = mul_w16<DIR, 6>(v[7]);
    const cpx b0 = v[0], b1 = v[2], b2 = v[4], b3 = v[6];
    v[0] = cadd(b0, w0); v[1] = cadd(b1, w1); v[2] = cadd(b2, w2); v[3] = cadd(b3, w3);
    v[4] = csub(b0, w0); v[5] = csub(b1, w1); v[6] = csub(b2, w2); v[7] = csub(b3, w3);
}

// First eight bins of a 16-point DFT:  out[c] = sum_{t<16} u[t] w16^(t c), c = 0..7.
template <int DIR> TFNO_DEV void dft16_first8(const cpx (&u)[16], cpx (&out)[8])
{
    // t = 2 t1 + t0:  out[c] = E[c] + w16^c O[c], E / O = 8-point transforms of the even / odd samples
    cpx e[8], o[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { e[i] = u[2 * i]; o[i] = u[2 * i + 1]; }
    fft8<DIR>(e);
    fft8<DIR>(o);
    out[0] = cadd(e[0], o[0]);                    out[1] = cadd(e[1], mul_w16<DIR, 1>(o[1]));
    out[2] = cadd(e[2], mul_w16<DIR, 2>(o[2]));   out[3] = cadd(e[3], mul_w16<DIR, 3>(o[3]));
    out[4] = cadd(e[4], mul_w16<DIR, 4>(o[4]));   out[5] = cadd(e[5], mul_w16<DIR, 5>(o[5]));
    out[6] = cadd(e[6], mul_w16<DIR, 6>(o[6]));   out[7] = cadd(e[7], mul_w16<DIR, 7>(o[7]));
}

// 16-point DFT of an 8-element input padded with 8 zeros:  h[t] = sum_{c<8} c[c] w16^(t c), t = 0..15.
template <int DIR> TFNO_DEV void dft16_pad8(const cpx (&c)[8], cpx (&h)[16])
{
    // c = 2 s + c0:  h[j] = H0[j] + w16^j H1[j],  h[j + 8] = H0[j] - w16^j H1[j],  H = 8-point pad transforms of even / odd inputs
    cpx ce[4], co[4], h0[8], h1[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) { ce[i] = c[2 * i]; co[i] = c[2 * i + 1]; }
    dft8_pad4<DIR>(ce, h0);
    dft8_pad4<DIR>(co, h1);
    const cpx w[8] = { h1[0], mul_w16<DIR, 1>(h1[1]), mul_w16<DIR, 2>(h1[2]), mul_w16<DIR, 3>(h1[3]),
                       mul_w16<DIR, 4>(h1[4]), mul_w16<DIR, 5>(h1[5]), mul_w16<DIR, 6>(h1[6]), mul_w16<DIR, 7>(h1[7]) };
#pragma unroll
    for (int j = 0; j < 8; ++j) { h[j] = cadd(h0[j], w[j]); h[j + 8] = csub(h0[j], w[j]); }
}

// Per-lane inter-pass twiddles  tw[r] = w_D^(t r), r = 0..15, for lane t of an L-lane group (D = 16 L).
template <int LOGD> TFNO_DEV void load_lane_twiddles(int t, cpx (&tw)[16])
{
#pragma unroll
    for (int r = 0; r < 16; ++r) tw[r] = kTwiddle1024[((t * r) << (10 - LOGD)) & 1023];
}

// Inter-pass twiddles kept in LDS instead of registers (frees 30 VGPRs for kernels that run 16 waves
// per CU). Table layout: tab[t*18 + r] = w_D^(t r), t < 16 lanes, r < 16; the pitch of 18 complex keeps
// 16-byte alignment for ds_read_b128 and spreads the 16 lanes of a group over all 64 banks.
constexpr int kTwLdsPitch = 18;
constexpr int kTwLdsSize = 16 * kTwLdsPitch;   // complex elements

#ifdef __HIPCC__
template <int LOGD, int ROWS = 16> TFNO_DEV void fill_lds_twiddles(cpx* tab, int tid, int nthreads)
{
    // all 16 lane rows (groups of fewer lanes use the first ones); ROWS = 32 / 64 for the lane groups of lengths 512 / 1024
    for (int e = tid; e < 16 * ROWS; e += nthreads) {
        const int t = e >> 4, r = e & 15;
        tab[t * kTwLdsPitch + r] = kTwiddle1024[((t * r) << (10 - LOGD)) & 1023];
    }
}
#endif

// Forward first pass with LDS twiddles: row = tab + t*kTwLdsPitch for lane t.
TFNO_DEV void fwd_pass1_lds(cpx (&v)[16], const cpx* row, cpx (&g)[16])
{
    fft16<-1>(v);
    g[0] = v[0];
#pragma unroll
    for (int r = 2; r < 16; r += 2) {
        const float4 w = *reinterpret_cast<const float4*>(row + r);      // tw[r], tw[r+1]
        g[r] = cmul(v[fft16_slot(r)], make_float2(w.x, w.y));
        g[r + 1] = cmul(v[fft16_slot(r + 1)], make_float2(w.z, w.w));
    }
    g[1] = cmul(v[fft16_slot(1)], row[1]);
}

// Second half of fwd_pass1_lds for a caller that ran fft16_stage1 itself: b[] in, twiddled bins out in g[].
TFNO_DEV void fwd_pass1_lds_finish(cpx (&b)[16], const cpx* row, cpx (&g)[16])
{
    fft16_stage2<-1>(b);
    g[0] = b[0];
#pragma unroll
    for (int r = 2; r < 16; r += 2) {
        const float4 w = *reinterpret_cast<const float4*>(row + r);      // tw[r], tw[r+1]
        g[r] = cmul(b[fft16_slot(r)], make_float2(w.x, w.y));
        g[r + 1] = cmul(b[fft16_slot(r + 1)], make_float2(w.z, w.w));
    }
    g[1] = cmul(b[fft16_slot(1)], row[1]);
}

// Backward last pass with LDS twiddles.
TFNO_DEV void inv_pass2_lds(cpx (&e)[16], const cpx* row, cpx (&y)[16])
{
#pragma unroll
    for (int r = 2; r < 16; r += 2) {
        const float4 w = *reinterpret_cast<const float4*>(row + r);
        e[r] = cmulc(e[r], make_float2(w.x, w.y));
        e[r + 1] = cmulc(e[r + 1], make_float2(w.z, w.w));
    }
    e[1] = cmulc(e[1], row[1]);
    fft16<+1>(e);
#pragma unroll
    for (int i = 0; i < 16; ++i) y[i] = e[fft16_slot(i)];
}

// Forward first pass: 16-point FFT of the lane's strided samples, then the inter-pass twiddle.
// On return g[r] (natural order) = w_D^(t r) * G_t[r].
TFNO_DEV void fwd_pass1(cpx (&v)[16], const cpx (&tw)[16], cpx (&g)[16])
{
    fft16<-1>(v);
#pragma unroll
    for (int r = 0; r < 16; ++r) g[r] = (r == 0) ? v[0] : cmul(v[fft16_slot(r)], tw[r]);
}

// Backward last pass: conj twiddle, 16-point backward FFT. e[r] in natural order; on return
// y[i] = value of output sample t + L*i.
TFNO_DEV void inv_pass2(cpx (&e)[16], const cpx (&tw)[16], cpx (&y)[16])
{
#pragma unroll
    for (int r = 1; r < 16; ++r) e[r] = cmulc(e[r], tw[r]);
    fft16<+1>(e);
#pragma unroll
    for (int i = 0; i < 16; ++i) y[i] = e[fft16_slot(i)];
}

// Lengths 512 and 1024 (L = 32 or 64 lanes per signal). After the exchange E[tt][r] (tt < L lanes, r < 16: first-pass
// results, already twiddled) the retained modes are  X[r + 16 c] = sum_{tt<L} E[tt][r] w_L^(tt c),  c < 4.  Split
// tt = a + A b with A = L/16 (2 or 4) and b < 16:
//     inner_a[c]  = sum_b E[a + A b][r] w16^(b c)       a pruned 16-point transform (dft16_first4), one (a, r) per lane
//     X[r + 16 c] = sum_{a<A} w_L^(a c) inner_a[c]      the A lanes of one r swap their inner values (a second, small
//                                                       exchange of 4 values per lane) and each finishes 4 / A modes
// i.e. 16 + 4 exchange reads and ~150 flops per lane instead of the L reads and L complex multiply-adds of a direct sum.
// Second-pass lane l = A r + a  (r = l / A, a = l % A) ends up with modes wide_mode<L>(l, j), j < 4 / A.
// `es` is the element stride of the exchange arrays (1 when a lane group has its own region; the number of columns
// when a block transforms several columns side by side).
template <int L> TFNO_DEV constexpr int wide_mode(int l, int j) { return (l / (L / 16)) + 16 * ((l % (L / 16)) * (64 / L) + j); }
// where lane (a', r) parks inner_a'[c] for the lane that finishes c
template <int L> TFNO_DEV constexpr int wide_swap_index(int r, int c, int a) { return (r * 4 + c) * (L / 16) + a; }

template <int L> TFNO_DEV void wide_forward_inner(const cpx* exch, int es, int l, cpx (&inner)[4])
{
    constexpr int A = L / 16;
    const int r = l / A, a = l % A;
    cpx u[16];
#pragma unroll
    for (int b = 0; b < 16; ++b) u[b] = exch[((a + A * b) * 17 + r) * es];
    dft16_first4<-1>(u, inner);
}
template <int L> TFNO_DEV void wide_forward_outer(const cpx* swap, int es, int l, cpx (&out)[64 / L])
{
    constexpr int A = L / 16, MM = 64 / L;
    const int r = l / A, a = l % A;
#pragma unroll
    for (int j = 0; j < MM; ++j) {
        const int c = a * MM + j;
        cpx acc = swap[wide_swap_index<L>(r, c, 0) * es];
#pragma unroll
        for (int ap = 1; ap < A; ++ap)
            cfma(acc, swap[wide_swap_index<L>(r, c, ap) * es], kTwiddle1024[(ap * c * (1024 / L)) & 1023]);
        out[j] = acc;
    }
}
// Backward: first-pass input r of lane t is  e[r] = sum_{c<4} C[r + 16 c] * conj(w_L^(t c)),  C = the 64 retained modes.
// With t = t1 + (L/4) t2 the factor splits into conj(w_L^(t1 c)) * i^(t2 c): lane l = (t1 = l % (L/4), rq = l / (L/4))
// twiddles the four modes C[r + 16 c] of r = rq + 4 ri, ri < 4, once (3 complex multiplications per r) and a 4-point
// transform without multiplications gives the inputs of the four lanes t2 < 4 at once. part[4 ri + t2] then belongs to
// lane t1 + (L/4) t2, slot r: the caller parks it at wide_back_index<L>(l, 4 ri + t2) of a pitch-17 array [L][17] (after
// every lane has read C, which may live in the same array) and each lane reads its e[r] back from row t. 16 + 16 + 16
// exchange accesses and ~110 flops per lane instead of 64 reads and ~290 flops for the direct sums.
template <int L>
TFNO_DEV void wide_backward_partial_tw(const cpx* c64, int es, int l, cpx w1, cpx w2, cpx w3, cpx (&part)[16])
{
    constexpr int Q = L / 4;
    const int rq = l / Q;
#pragma unroll
    for (int ri = 0; ri < 4; ++ri) {
        const int r = rq + 4 * ri;
        const cpx d0 = c64[r * es], d1 = cmulc(c64[(r + 16) * es], w1), d2 = cmulc(c64[(r + 32) * es], w2),
                  d3 = cmulc(c64[(r + 48) * es], w3);
        const cpx s02 = cadd(d0, d2), m02 = csub(d0, d2), s13 = cadd(d1, d3), m13 = csub(d1, d3);
        const cpx im13 = make_float2(-m13.y, m13.x);            // i * (d1 - d3)
        part[4 * ri + 0] = cadd(s02, s13);
        part[4 * ri + 1] = cadd(m02, im13);
        part[4 * ri + 2] = csub(s02, s13);
        part[4 * ri + 3] = csub(m02, im13);
    }
}
template <int L> TFNO_DEV void wide_backward_partial(const cpx* c64, int es, int l, cpx (&part)[16])
{
    const int t1 = l % (L / 4);
    wide_backward_partial_tw<L>(c64, es, l, kTwiddle1024[(t1 * (1024 / L)) & 1023], kTwiddle1024[(2 * t1 * (1024 / L)) & 1023],
                                kTwiddle1024[(3 * t1 * (1024 / L)) & 1023], part);
}
template <int L> TFNO_DEV constexpr int wide_back_index(int l, int k)
{
    return ((l % (L / 4)) + (L / 4) * (k & 3)) * 17 + (l / (L / 4)) + 4 * (k >> 2);
}

// Orders LDS traffic of one wavefront: everything the wave wrote before is visible to its own
// lanes after. DS operations of a wave complete in issue order, so no hardware wait is needed
// beyond what the compiler inserts for the data dependency; this only stops compiler reordering.
#ifdef __HIPCC__
// Streaming (non-temporal) global accesses for data touched exactly once.
typedef float tfno_v2f __attribute__((ext_vector_type(2)));
TFNO_DEV cpx load_streaming(const cpx* p)
{
    const tfno_v2f v = __builtin_nontemporal_load(reinterpret_cast<const tfno_v2f*>(p));
    return make_float2(v.x, v.y);
}
TFNO_DEV void store_streaming(cpx* p, cpx v)
{
    tfno_v2f q = { v.x, v.y };
    __builtin_nontemporal_store(q, reinterpret_cast<tfno_v2f*>(p));
}

TFNO_DEV void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
#else
// Host builds (CPU checks of the group transforms): the lanes of a group are threads there, and the check supplies
// the point at which all of them have arrived.
void wave_lds_fence();
#endif

}  // namespace tfno
