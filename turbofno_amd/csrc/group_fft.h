// Transforms of one signal by one L-lane group of a wavefront (L = D/16 lanes, 16 samples per lane; L = 8, 16 for
// lengths 128, 256 and, with a pruned second pass in two steps, L = 32, 64 for lengths 512, 1024), built from the register
// codelets plus one padded LDS exchange that stays inside the wavefront (no block barrier). Shared by the fused 1D kernel and the 2D image kernels.
#pragma once
#include "fft_codelets.h"

namespace tfno {

template <int LOGDY> struct Geo1D {
    static constexpr int DY = 1 << LOGDY;
    static constexpr int L = DY / 16;        // lanes per signal
    static constexpr int GROUPS = 256 / L;   // signals transformed concurrently = K chunk
    static constexpr int MM = 64 / L;        // modes owned per lane   (m = lane + L*mm)
    static constexpr int NN = 64 / GROUPS;   // output channels per group (n = g + GROUPS*jn)
    static constexpr int EXCH = L * 17;      // complex per group exchange region
    // pitches (complex) of the spectra tile sA[kk][m] and the weight tile sW[kk][n] of the fused kernel: rows of sA are
    // written by neighbouring lane groups at once (80: half the banks apart), rows of sW by consecutive lanes (65)
    static constexpr int SA_PITCH = 80, SW_PITCH = 65;
    static constexpr size_t LDS_BYTES = sizeof(float2) * (size_t)(GROUPS * SA_PITCH + GROUPS * SW_PITCH + GROUPS * EXCH);
};

// Lengths 512 / 1024: a group of L = 32 / 64 lanes owns one signal, lane t holds samples t + L i. The scheme of the wide_*
// codelets (inner 16-point transforms over the lanes tt = a + A b, A = L / 16, then a sum over a), with the lanes and the
// two exchanges laid out for the LDS banks (64 banks of 4 bytes, 32 lanes of 8 bytes per cycle):
//   second-pass lane t = 16 a + r computes inner_a[c] of bin r, then finishes the modes r + 16 (a + A j) = t + L j: the
//     natural order, L consecutive modes per slot j;
//   first exchange: the A rows a + A b of one b side by side, [b][a][16 bins] with a pitch of 16 A + 1: the read of one b
//     covers 32 consecutive elements per half wavefront, the write of one bin is conflict-free for L = 32 (2-way for 64);
//   second exchange: [c][16 a' + r] with a pitch of L + 16: writes are consecutive, and the lanes a and a + 1 of a half
//     wavefront, which read the rows c = a + A j and c + 1, land 16 elements apart modulo 32.
// The powers w_L^e, e < L, come from the constant table, or (FROM_ARRAY) from an array of L values that the caller keeps
// in LDS where a global load would be in the way.
// g[]: first-pass results, already twiddled. On return out[j] = mode t + L j.
template <int L, bool FROM_ARRAY> TFNO_DEV cpx wide_pow(const cpx* powers, int e)
{
    if constexpr (FROM_ARRAY) return powers[e];
    else return kTwiddle1024[(e * (1024 / L)) & 1023];
}
template <int L, bool FROM_ARRAY>
TFNO_DEV void wide_forward_finish(const cpx (&g)[16], cpx* exch, const cpx* powers, int t, cpx (&out)[64 / L])
{
    constexpr int A = L / 16, MM = 64 / L, P1 = 16 * A + 1, PS = L + 16;
    static_assert(16 * P1 <= L * 17 && 4 * PS <= L * 17, "both exchanges fit the group's region");
    const int r = t % 16, a = t / 16;
    wave_lds_fence();
#pragma unroll
    for (int k = 0; k < 16; ++k) exch[(t / A) * P1 + (t % A) * 16 + k] = g[k];
    wave_lds_fence();
    cpx inner[4];
    {
        cpx u[16];
#pragma unroll
        for (int b = 0; b < 16; ++b) u[b] = exch[b * P1 + t];      // lane tt = a + A b, bin r
        dft16_first4<-1>(u, inner);
    }
    wave_lds_fence();                                // every lane of the group has read the first exchange
#pragma unroll
    for (int c = 0; c < 4; ++c) exch[c * PS + t] = inner[c];
    wave_lds_fence();
#pragma unroll
    for (int j = 0; j < MM; ++j) {
        const int c = a + A * j;
        cpx acc = exch[c * PS + r];
#pragma unroll
        for (int ap = 1; ap < A; ++ap) cfma(acc, exch[c * PS + 16 * ap + r], wide_pow<L, FROM_ARRAY>(powers, (ap * c) % L));
        out[j] = acc;
    }
}

// Backward, up to the inputs of the last pass: c[mm] = mode t + L mm; on return e[r] = first-pass input r of lane t
// (before the conjugate twiddle). Lane l = (t1 = l % Q, rq = l / Q), Q = L / 4, forms the inputs of the four lanes
// t1 + Q t2 for the bins r = rq + 4 ri (wide_backward_partial_tw) and parks them for their owners at
// [r][lane ^ (Q rq)], rows of L: the owners read a row as L consecutive elements, and the XOR puts the four rq of one
// write Q elements apart, so that the 32 lanes of a half wavefront hit 32 different bank pairs in both directions.
template <int L, bool FROM_ARRAY>
TFNO_DEV void wide_backward_inputs(const cpx (&c)[64 / L], const cpx* powers, cpx* exch, int t, cpx (&e)[16])
{
    constexpr int Q = L / 4;
    wave_lds_fence();
#pragma unroll
    for (int mm = 0; mm < 64 / L; ++mm) exch[t + L * mm] = c[mm];
    wave_lds_fence();
    cpx part[16];
    const int t1 = t % Q, rq = t / Q;
    wide_backward_partial_tw<L>(exch, 1, t, wide_pow<L, FROM_ARRAY>(powers, t1), wide_pow<L, FROM_ARRAY>(powers, 2 * t1),
                                wide_pow<L, FROM_ARRAY>(powers, 3 * t1), part);
    wave_lds_fence();                                // every lane of the group has read the 64 modes
#pragma unroll
    for (int ri = 0; ri < 4; ++ri)
#pragma unroll
        for (int t2 = 0; t2 < 4; ++t2) exch[(rq + 4 * ri) * L + t1 + Q * (t2 ^ rq)] = part[4 * ri + t2];
    wave_lds_fence();
#pragma unroll
    for (int r = 0; r < 16; ++r) e[r] = exch[r * L + (t ^ (Q * (r & 3)))];
}
// Mode that lane t of an L-lane group holds in out[mm] after a forward transform.
template <int LOGDY> TFNO_DEV constexpr int forward_mode_of_lane(int t, int mm)
{
    constexpr int L = (1 << LOGDY) / 16;
    return t + L * mm;
}

// second half of the forward transform: exchange of the twiddled first-pass results g[] inside the
// L-lane group, then the pruned L-point DFT. On return lane `t` holds mode forward_mode_of_lane<LOGDY>(t, mm) =
// t + L*mm in out[mm].
template <int LOGDY>
TFNO_DEV void group_forward_finish(const cpx (&g)[16], cpx* exch, int t, cpx (&out)[Geo1D<LOGDY>::MM])
{
    constexpr int L = Geo1D<LOGDY>::L;
    if constexpr (L >= 32) {
        wide_forward_finish<L, false>(g, exch, nullptr, t, out);
        return;
    }
    wave_lds_fence();
#pragma unroll
    for (int r = 0; r < 16; ++r) exch[t * 17 + r] = g[r];
    wave_lds_fence();
    if constexpr (L == 16) {
        cpx u[16];
#pragma unroll
        for (int tt = 0; tt < 16; ++tt) u[tt] = exch[tt * 17 + t];
        dft16_first4<-1>(u, out);                       // out[s] = X[t + 16 s]
    } else if constexpr (L == 8) {
        cpx u0[8], u1[8], o0[4], o1[4];
#pragma unroll
        for (int tt = 0; tt < 8; ++tt) { u0[tt] = exch[tt * 17 + t]; u1[tt] = exch[tt * 17 + t + 8]; }
        dft8_first4<-1>(u0, o0);                        // X[t + 16 s]
        dft8_first4<-1>(u1, o1);                        // X[t + 8 + 16 s]
#pragma unroll
        for (int s = 0; s < 4; ++s) { out[2 * s] = o0[s]; out[2 * s + 1] = o1[s]; }
    }
}

// forward transform of one signal by one L-lane group; lane t holds samples t + L*i in v[].
// On return lane `t` holds mode forward_mode_of_lane<LOGDY>(t, mm) in out[mm].
template <int LOGDY>
TFNO_DEV void group_forward(cpx (&v)[16], const cpx (&tw)[16], cpx* exch, int t, cpx (&out)[Geo1D<LOGDY>::MM])
{
    cpx g[16];
    fwd_pass1(v, tw, g);
    group_forward_finish<LOGDY>(g, exch, t, out);
}

// zero-padded backward transform; lane t holds modes m = t + L*mm in c[]; returns samples t + L*i in y[].
template <int LOGDY>
TFNO_DEV void group_backward(const cpx (&c)[Geo1D<LOGDY>::MM], const cpx (&tw)[16], cpx* exch, int t, cpx (&y)[16])
{
    constexpr int L = Geo1D<LOGDY>::L;
    cpx e[16];
    if constexpr (L >= 32) {
        wide_backward_inputs<L, false>(c, nullptr, exch, t, e);
    } else {
        wave_lds_fence();
        if constexpr (L == 16) {
            cpx h[16];
            dft16_pad4<+1>(c, h);
#pragma unroll
            for (int tt = 0; tt < 16; ++tt) exch[tt * 17 + t] = h[tt];
        } else {
            cpx c0[4], c1[4], h0[8], h1[8];
#pragma unroll
            for (int s = 0; s < 4; ++s) { c0[s] = c[2 * s]; c1[s] = c[2 * s + 1]; }
            dft8_pad4<+1>(c0, h0);
            dft8_pad4<+1>(c1, h1);
#pragma unroll
            for (int tt = 0; tt < 8; ++tt) { exch[tt * 17 + t] = h0[tt]; exch[tt * 17 + t + 8] = h1[tt]; }
        }
        wave_lds_fence();
#pragma unroll
        for (int r = 0; r < 16; ++r) e[r] = exch[t * 17 + r];
    }
    inv_pass2(e, tw, y);
}

// zero-padded backward transform whose last pass takes its twiddles from an LDS table row
// (twrow = table + t * kTwLdsPitch). Lane t holds modes m = t + L*mm in c[]; returns samples t + L*i in y[].
template <int LOGD>
TFNO_DEV void group_backward_lds(const cpx (&c)[Geo1D<LOGD>::MM], const cpx* twrow, cpx* exch, int t, cpx (&y)[16])
{
    constexpr int L = Geo1D<LOGD>::L;
    wave_lds_fence();
    static_assert(L <= 16, "the whole-image kernels are built for lengths 128 and 256");
    if constexpr (L == 16) {
        cpx h[16];
        dft16_pad4<+1>(c, h);
#pragma unroll
        for (int tt = 0; tt < 16; ++tt) exch[tt * 17 + t] = h[tt];
    } else {
        cpx c0[4], c1[4], h0[8], h1[8];
#pragma unroll
        for (int s = 0; s < 4; ++s) { c0[s] = c[2 * s]; c1[s] = c[2 * s + 1]; }
        dft8_pad4<+1>(c0, h0);
        dft8_pad4<+1>(c1, h1);
#pragma unroll
        for (int tt = 0; tt < 8; ++tt) { exch[tt * 17 + t] = h0[tt]; exch[tt * 17 + t + 8] = h1[tt]; }
    }
    wave_lds_fence();
    cpx e[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) e[r] = exch[t * 17 + r];
    inv_pass2_lds(e, twrow, y);
}

// Rows of 128 in the whole-image kernels: a 16-lane group owns TWO rows, lane t holds samples t + 16 i (i < 8) of
// each, so a group still moves 128 contiguous bytes per load or store. The first pass is a pair of 8-point FFTs;
// after the exchange lane t = r + 8 h finishes row h: modes r + 8 c, c < 8. Twiddles w_128^(t r) come from the lane's
// row of the LDS table.
#ifdef __HIPCC__
// g[0..7] / g[8..15]: first-pass results of row A / row B, already twiddled. On return out[c] = mode (t & 7) + 8 c
// of row (t >> 3).
TFNO_DEV void rows128_forward_finish(const cpx (&g)[16], cpx* exch, int t, cpx (&out)[8])
{
    wave_lds_fence();
#pragma unroll
    for (int j = 0; j < 16; ++j) exch[t * 17 + j] = g[j];
    wave_lds_fence();
    cpx u[16];
#pragma unroll
    for (int tt = 0; tt < 16; ++tt) u[tt] = exch[tt * 17 + t];
    dft16_first8<-1>(u, out);
}

// c[k] = mode (t & 7) + 8 k of row (t >> 3). On return y[i] / y[8 + i] = sample t + 16 i of row A / row B.
template <class TW>   // twrow[r] = w_128^(t r), r < 8: a row of the LDS table or a register array
TFNO_DEV void rows128_backward(const cpx (&c)[8], const TW& twrow, cpx* exch, int t, cpx (&y)[16])
{
    cpx h[16];
    dft16_pad8<+1>(c, h);
    wave_lds_fence();
#pragma unroll
    for (int tt = 0; tt < 16; ++tt) exch[tt * 17 + t] = h[tt];
    wave_lds_fence();
    cpx a[8], b[8];
    a[0] = exch[t * 17];
    b[0] = exch[t * 17 + 8];
#pragma unroll
    for (int r = 1; r < 8; ++r) {
        const cpx w = twrow[r];
        a[r] = cmulc(exch[t * 17 + r], w);
        b[r] = cmulc(exch[t * 17 + 8 + r], w);
    }
    fft8<+1>(a);
    fft8<+1>(b);
#pragma unroll
    for (int i = 0; i < 8; ++i) { y[i] = a[i]; y[8 + i] = b[i]; }
}

// Rows of 512 / 1024 in the whole-image kernels: wide_forward_finish / wide_backward_inputs with every twiddle taken
// from LDS (a global load inside the row loop would queue behind the loads of the next row, which are in flight all
// the time): twrow = the lane's row of the first-pass table, wsm[e] = w_L^e, e < L.
template <int L>
TFNO_DEV void wide_rows_forward_finish(const cpx (&g)[16], cpx* exch, const cpx* wsm, int t, cpx (&out)[64 / L])
{
    wide_forward_finish<L, true>(g, exch, wsm, t, out);
}
// c[mm] = mode t + L mm of the row. On return y[i] = sample t + L i.
template <int L>
TFNO_DEV void wide_rows_backward(const cpx (&c)[64 / L], const cpx* twrow, const cpx* wsm, cpx* exch, int t, cpx (&y)[16])
{
    cpx e[16];
    wide_backward_inputs<L, true>(c, wsm, exch, t, e);
    inv_pass2_lds(e, twrow, y);
}

// The same pairing for the 1D kernels, with the twiddles in registers (tw[r] = w_128^(t r), t < 16): a 16-lane group
// transforms two signals; v[0..7] / v[8..15] are samples t + 16 i of signal A / signal B. On return out[c] is mode
// (t & 7) + 8 c of signal (t >> 3): the lane-to-mode mapping of an 8-lane group per signal, so callers index their
// tiles as for L = 8 and only the loads and stores change to 128-byte segments.
TFNO_DEV void pair128_forward(const cpx (&v)[16], const cpx (&tw)[16], cpx* exch, int t, cpx (&out)[8])
{
    cpx a[8], b[8], g[16];
#pragma unroll
    for (int i = 0; i < 8; ++i) { a[i] = v[i]; b[i] = v[8 + i]; }
    fft8<-1>(a);
    fft8<-1>(b);
    g[0] = a[0];
    g[8] = b[0];
#pragma unroll
    for (int r = 1; r < 8; ++r) { g[r] = cmul(a[r], tw[r]); g[8 + r] = cmul(b[r], tw[r]); }
    rows128_forward_finish(g, exch, t, out);
}
// c[k] = mode (t & 7) + 8 k of signal (t >> 3); on return y[i] / y[8 + i] = sample t + 16 i of signal A / signal B.
TFNO_DEV void pair128_backward(const cpx (&c)[8], const cpx (&tw)[16], cpx* exch, int t, cpx (&y)[16])
{
    rows128_backward(c, tw, exch, t, y);
}

// The 16 samples t + L i of one output signal. By default y is streamed past the caches (it is written once and not read
// again by the layer); KEEP leaves it cached for a consumer that follows at once (the X-axis backward kernel of the
// three-kernel 2D pipeline: 895 -> 854 us for 16 images of 512 x 512, K = 32, N = 64).
template <int L, bool KEEP> TFNO_DEV void store_row16(float2* dst, const cpx (&yv)[16])
{
    if constexpr (KEEP) {
#pragma unroll
        for (int i = 0; i < 16; ++i) dst[L * i] = yv[i];
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) store_streaming(dst + L * i, yv[i]);
    }
}

// The same for two signals handled by one 16-lane group (lengths of 128): samples t + 16 i of signal A in yv[i], of signal B
// (`second` elements further on) in yv[8 + i].
template <bool KEEP> TFNO_DEV void store_pair16(float2* dst, long second, const cpx (&yv)[16])
{
    if constexpr (KEEP) {
#pragma unroll
        for (int i = 0; i < 8; ++i) { dst[16 * i] = yv[i]; dst[second + 16 * i] = yv[8 + i]; }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) { store_streaming(dst + 16 * i, yv[i]); store_streaming(dst + second + 16 * i, yv[8 + i]); }
    }
}
#endif

}  // namespace tfno
