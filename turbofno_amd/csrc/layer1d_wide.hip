// Fused 1D spectral layer for LARGE grids with many channels (DY = 256, and DY = 128 further down): one 256-thread block per (signal set, NT output
// channels) with NT = 128 or 64, so that with N = 128 every input channel of a signal set is transformed once, not once
// per 64 output channels, and the contraction takes three real matrix instructions per complex product instead of four.
//
// Same operands and result as fused_fft_cgemm_ifft_8 of the reference
// (fusion_variants/1D_D_exp_fused_fft_cgemm_ifft/fused_fft_cgemm_ifft_7.cuh:9-222: (S, N/64) blocks that each traverse
// K). Per chunk of 16 channels (one per 16-lane group): forward transforms -> spectra tile sA[16][64] in LDS; the rows
// of W for ALL NT output channels -> W'' tile, three planes (c, d - c, c + d with alpha W = c + i d) in the bank-conflict
// free order of the mode GEMM; wave w owns the 16 modes 16 w ... 16 w + 15 and NT / 16 tiles of 16 output channels,
// three accumulator tiles each (P1 = c (a + b), P2 = (d - c) a, P3 = (c + d) b; re = P1 - P3, im = P1 + P2), kept in
// registers across the chunks. After the K loop the product goes to LDS 16 channels at a time (two buffers in the
// region the W'' tile no longer needs) and the 16 lane groups run the zero-padded backward transforms.
// LDS 62 KiB: two blocks per CU, which are in different phases most of the time, so that the loads, the vector work
// and the matrix work of the two overlap.
#include "group_fft.h"
#include "kernels.h"

namespace tfno {

typedef float floatx4_w __attribute__((ext_vector_type(4)));

template <int NT> struct GeoWide {
    static constexpr int KC = 16;                               // channels per chunk = lane groups of a block
    static constexpr int PA = 80, PC = 72;                      // pitches (complex) of the spectra tile and of the product buffers
    static constexpr int EXCH = 16 * 17;
    static constexpr int REGION0 = KC * EXCH;                   // exchange regions | spectra tile sA[KC][PA]
    static constexpr int WROW = NT + 16, WGROUP = 4 * WROW + 1, WPLANE = (KC / 4) * WGROUP;
    static constexpr int WTILE = (3 * WPLANE + 1) / 2;          // complex units
    static constexpr int REGION1 = WTILE > 2 * 16 * PC ? WTILE : 2 * 16 * PC;   // W'' tile | two product buffers sC[2][16][PC]
    static constexpr int TILES = NT / 16;                       // tiles of 16 output channels per wave
    static constexpr size_t LDS_BYTES = sizeof(float2) * (size_t)(REGION0 + REGION1);
    static_assert(KC * PA <= REGION0, "spectra tile must fit the exchange regions");
    static_assert(WROW % 64 == 16, "rows of an operand fetch must be 16 banks apart");
};

template <int NT, bool KEEP>
__global__ __launch_bounds__(256, 2) void fused_fft_mfma_ifft_wide_kernel(int S, int N, int K, const float2* __restrict__ x,
                                                                         const float2* __restrict__ W, float2* __restrict__ y,
                                                                         float2 alpha)
{
    using G = GeoWide<NT>;
    constexpr int DY = 256, KC = G::KC, PA = G::PA, PC = G::PC, TILES = G::TILES;
    extern __shared__ float2 lds[];
    float2* sA = lds;
    float* sW = reinterpret_cast<float*>(lds + G::REGION0);
    float2* sC = lds + G::REGION0;

    const int tid = threadIdx.x;
    const int g = tid >> 4, t = tid & 15;                       // transform role: lane group g, lane t
    const int mt = tid >> 6, lane = tid & 63, col = lane & 15, kq = lane >> 4;     // matrix role: m tile = wave
    long s;
    int ntile;
    decode_block_1d(S, N / NT, 256, !KEEP, s, ntile);
    const int n0 = ntile * NT;
    float2* exch = lds + g * G::EXCH;

    cpx tw[16];
    load_lane_twiddles<8>(t, tw);
    floatx4_w p1[TILES], p2[TILES], p3[TILES];
#pragma unroll
    for (int i = 0; i < TILES; ++i) p1[i] = p2[i] = p3[i] = floatx4_w{ 0.f, 0.f, 0.f, 0.f };

    const float2* src = x + ((long)g * S + s) * DY + t;
    auto issue = [&](cpx (&dst)[16], int kc) {
        const float2* p = src + (long)kc * S * DY;
#pragma unroll
        for (int i = 0; i < 16; ++i) dst[i] = p[16 * i];
    };
    // one chunk of loads in flight per lane group, refilled as soon as the first pass has consumed it (a second buffer
    // needs the inter-pass twiddles in LDS to fit the registers and was measured slower: 0-4 % with 64-channel tiles,
    // spills with 128-channel tiles)
    cpx v[16];
    if (g < K) issue(v, 0);

    for (int kc = 0; kc < K; kc += KC) {
        const int kn = (K - kc) < KC ? (K - kc) : KC;           // 16, or 8 in the last chunk (K is a multiple of 8)
        // W chunk: lanes run along k, the contiguous direction of W[k + n*K]; the four channels n a wavefront touches in
        // one instruction are four apart (four banks apart in the tile)
        constexpr int WPT = KC * NT / 256;
        float2 wv[WPT];
#pragma unroll
        for (int u = 0; u < WPT; ++u) {
            const int idx = tid + u * 256;
            const int k = idx % KC, r = idx / KC, n = (r & ~15) | ((r & 3) << 2) | ((r >> 2) & 3);
            wv[u] = (k < kn) ? W[(kc + k) + (long)(n0 + n) * K] : make_float2(0.f, 0.f);
        }
        cpx out[4];
        if (g < kn) {
            cpx gg[16];
            fwd_pass1(v, tw, gg);
            if (kc + KC + g < K) issue(v, kc + KC);
            group_forward_finish<8>(gg, exch, t, out);
        } else {
#pragma unroll
            for (int a = 0; a < 4; ++a) out[a] = make_float2(0.f, 0.f);
        }
        // W'' tile (its region is not shared with the transforms): built by whichever waves are done transforming
#pragma unroll
        for (int u = 0; u < WPT; ++u) {
            const int idx = tid + u * 256;
            const int k = idx % KC, r = idx / KC, n = (r & ~15) | ((r & 3) << 2) | ((r >> 2) & 3);
            const float c = wv[u].x * alpha.x - wv[u].y * alpha.y, d = wv[u].x * alpha.y + wv[u].y * alpha.x;
            float* dstw = &sW[(k >> 2) * G::WGROUP + (k & 3) * G::WROW + n];
            dstw[0] = c;
            dstw[G::WPLANE] = d - c;
            dstw[2 * G::WPLANE] = c + d;
        }
        __syncthreads();                                        // all exchanges done: sA may overwrite them
#pragma unroll
        for (int a = 0; a < 4; ++a) sA[g * PA + t + 16 * a] = out[a];   // zeros beyond a short last chunk
        __syncthreads();
        const float2* arow = sA + kq * PA + mt * 16 + col;
        float2 b[KC / 4];
#pragma unroll
        for (int kg = 0; kg < KC / 4; ++kg) b[kg] = arow[kg * 4 * PA];
#pragma unroll
        for (int i = 0; i < TILES; ++i) {
            const float* wrow = sW + kq * G::WROW + i * 16 + col;
#pragma unroll
            for (int kg = 0; kg < KC / 4; ++kg) {
                const float* w = wrow + kg * G::WGROUP;
                p1[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[0], b[kg].x + b[kg].y, p1[i], 0, 0, 0);
                p2[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[G::WPLANE], b[kg].x, p2[i], 0, 0, 0);
                p3[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[2 * G::WPLANE], b[kg].y, p3[i], 0, 0, 0);
            }
        }
        __syncthreads();                                        // sA / sW are free again (next chunk, or the product below)
    }

    // D[row = 4 kq + v][col] of tile i: output channel n0 + 16 i + 4 kq + v, mode 16 mt + col. Tile i goes to product
    // buffer i & 1; lane group g then transforms channel n0 + 16 i + g. One barrier per tile: buffer i & 1 was last read
    // in step i - 2, which every wave has left before the barrier of step i - 1.
#pragma unroll
    for (int i = 0; i < TILES; ++i) {
        float2* buf = sC + (i & 1) * 16 * PC;
#pragma unroll
        for (int vv = 0; vv < 4; ++vv)
            buf[(4 * kq + vv) * PC + mt * 16 + col] = make_float2(p1[i][vv] - p3[i][vv], p1[i][vv] + p2[i][vv]);
        __syncthreads();
        cpx c[4], yv[16];
#pragma unroll
        for (int a = 0; a < 4; ++a) c[a] = buf[g * PC + t + 16 * a];
        group_backward<8>(c, tw, exch, t, yv);
        float2* dst = y + ((long)(n0 + 16 * i + g) * S + s) * DY + t;
        store_row16<16, KEEP>(dst, yv);
    }
}

// The same for DY = 128, where a 16-lane group transforms two channels at a time (pair128_forward / _backward), so that a
// round of the block covers 32 channels: the spectra tile holds 32 channels, the W'' tile 16 - it is built and multiplied
// twice per round, and the rows of W for the second half are fetched while the first half is being multiplied. The
// product goes to LDS 32 channels at a time.
template <int NT, bool KEEP>
__global__ __launch_bounds__(256, 2) void fused_fft_mfma_ifft_wide128_kernel(int S, int N, int K, const float2* __restrict__ x,
                                                                            const float2* __restrict__ W, float2* __restrict__ y,
                                                                            float2 alpha)
{
    using G = GeoWide<NT>;
    constexpr int DY = 128, PA = G::PA, PC = G::PC, TILES = G::TILES, KR = 32;    // KR = channels per round
    static_assert(KR * PA <= G::REGION0 && KR * PC <= G::REGION1, "32-channel tiles must fit the regions");
    extern __shared__ float2 lds[];
    float2* sA = lds;
    float* sW = reinterpret_cast<float*>(lds + G::REGION0);
    float2* sC = lds + G::REGION0;

    const int tid = threadIdx.x;
    const int grp = tid >> 4, t16 = tid & 15;                   // transform role: 16-lane group, two channels each
    const int g8 = tid >> 3, r8 = tid & 7;                      // after the exchange: lane r8 of channel g8 of the round
    const int mt = tid >> 6, lane = tid & 63, col = lane & 15, kq = lane >> 4;     // matrix role: m tile = wave
    long s;
    int ntile;
    decode_block_1d(S, N / NT, 128, !KEEP, s, ntile);
    const int n0 = ntile * NT;
    float2* exch = lds + grp * G::EXCH;

    cpx tw[16];
    load_lane_twiddles<7>(t16, tw);
    floatx4_w p1[TILES], p2[TILES], p3[TILES];
#pragma unroll
    for (int i = 0; i < TILES; ++i) p1[i] = p2[i] = p3[i] = floatx4_w{ 0.f, 0.f, 0.f, 0.f };

    const float2* src = x + ((long)(2 * grp) * S + s) * DY + t16;
    auto issue = [&](cpx (&dst)[16], int kc) {
        const float2* p = src + (long)kc * S * DY;
#pragma unroll
        for (int i = 0; i < 8; ++i) { dst[i] = p[16 * i]; dst[8 + i] = p[(long)S * DY + 16 * i]; }
    };
    cpx v[16];
    if (2 * grp < K) issue(v, 0);

    constexpr int WPT = 16 * NT / 256;
    auto load_w = [&](float2 (&wv)[WPT], int k0, int kn) {      // rows k0 ... k0 + 15 of W, zeros from row kn of the round on
#pragma unroll
        for (int u = 0; u < WPT; ++u) {
            const int idx = tid + u * 256;
            const int k = idx % 16, r = idx / 16, n = (r & ~15) | ((r & 3) << 2) | ((r >> 2) & 3);
            wv[u] = (k0 % KR + k < kn) ? W[(k0 + k) + (long)(n0 + n) * K] : make_float2(0.f, 0.f);
        }
    };
    auto build_w = [&](const float2 (&wv)[WPT]) {
#pragma unroll
        for (int u = 0; u < WPT; ++u) {
            const int idx = tid + u * 256;
            const int k = idx % 16, r = idx / 16, n = (r & ~15) | ((r & 3) << 2) | ((r >> 2) & 3);
            const float c = wv[u].x * alpha.x - wv[u].y * alpha.y, d = wv[u].x * alpha.y + wv[u].y * alpha.x;
            float* dstw = &sW[(k >> 2) * G::WGROUP + (k & 3) * G::WROW + n];
            dstw[0] = c;
            dstw[G::WPLANE] = d - c;
            dstw[2 * G::WPLANE] = c + d;
        }
    };
    auto multiply = [&](int half) {                             // channels 16 half ... 16 half + 15 of the round
        const float2* arow = sA + (16 * half + kq) * PA + mt * 16 + col;
        float2 b[4];
#pragma unroll
        for (int kg = 0; kg < 4; ++kg) b[kg] = arow[kg * 4 * PA];
#pragma unroll
        for (int i = 0; i < TILES; ++i) {
            const float* wrow = sW + kq * G::WROW + i * 16 + col;
#pragma unroll
            for (int kg = 0; kg < 4; ++kg) {
                const float* w = wrow + kg * G::WGROUP;
                p1[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[0], b[kg].x + b[kg].y, p1[i], 0, 0, 0);
                p2[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[G::WPLANE], b[kg].x, p2[i], 0, 0, 0);
                p3[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[2 * G::WPLANE], b[kg].y, p3[i], 0, 0, 0);
            }
        }
    };

    for (int kc = 0; kc < K; kc += KR) {
        const int kn = (K - kc) < KR ? (K - kc) : KR;           // 8, 16, 24 or 32 (K is a multiple of 8)
        float2 wv[WPT];
        load_w(wv, kc, kn);
        cpx out[8];
        if (2 * grp < kn) {
            cpx w[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) w[i] = v[i];
            if (kc + KR + 2 * grp < K) issue(v, kc + KR);
            pair128_forward(w, tw, exch, t16, out);
        } else {
#pragma unroll
            for (int c = 0; c < 8; ++c) out[c] = make_float2(0.f, 0.f);
        }
        build_w(wv);
        if (kn > 16) load_w(wv, kc + 16, kn);                   // second half of the rows: arrives under the first multiply
        __syncthreads();                                        // all exchanges done: sA may overwrite them
#pragma unroll
        for (int c = 0; c < 8; ++c) sA[g8 * PA + r8 + 8 * c] = out[c];     // zeros beyond a short last round
        __syncthreads();
        multiply(0);
        if (kn > 16) {                                          // uniform
            __syncthreads();                                    // the first half of the W'' tile is consumed
            build_w(wv);
            __syncthreads();
            multiply(1);
        }
        __syncthreads();                                        // sA / sW are free again (next round, or the product below)
    }

    // product -> LDS 32 channels (two tiles) at a time; lane (g8, r8) takes modes r8 + 8 k of channel 32 step + g8
#pragma unroll
    for (int step = 0; step < TILES / 2; ++step) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int vv = 0; vv < 4; ++vv) {
                const int i = 2 * step + j;
                sC[(16 * j + 4 * kq + vv) * PC + mt * 16 + col] = make_float2(p1[i][vv] - p3[i][vv], p1[i][vv] + p2[i][vv]);
            }
        __syncthreads();
        cpx c[8], yv[16];
#pragma unroll
        for (int k = 0; k < 8; ++k) c[k] = sC[g8 * PC + r8 + 8 * k];
        __syncthreads();                                        // the buffer is consumed: the next step may overwrite it
        pair128_backward(c, tw, exch, t16, yv);
        float2* dst = y + ((long)(n0 + 32 * step + 2 * grp) * S + s) * DY + t16;
        store_pair16<KEEP>(dst, (long)S * DY, yv);
    }
}

template <int NT, bool KEEP>
static hipError_t launch_wide_t(int logDY, long S, int N, int K, const float2* x, const float2* W, float2* y, float2 alpha,
                                hipStream_t stream)
{
    using G = GeoWide<NT>;
    if (S * (N / NT) > 0x7fffffffL) return hipErrorInvalidValue;
    static_assert(G::LDS_BYTES <= 64 * 1024, "no attribute call needed below 64 KiB of dynamic LDS");
    if (logDY == 7)
        hipLaunchKernelGGL((fused_fft_mfma_ifft_wide128_kernel<NT, KEEP>), dim3((unsigned)(S * (N / NT))), dim3(256), G::LDS_BYTES, stream,
                           (int)S, N, K, x, W, y, alpha);
    else
        hipLaunchKernelGGL((fused_fft_mfma_ifft_wide_kernel<NT, KEEP>), dim3((unsigned)(S * (N / NT))), dim3(256), G::LDS_BYTES, stream,
                           (int)S, N, K, x, W, y, alpha);
    return hipGetLastError();
}

// DY = 128 or 256. Tiles of 128 output channels when N allows, else of 64.
hipError_t launch_fused_wide(int logDY, long S, int N, int K, const float2* x, const float2* W, float2* y, float2 alpha,
                             hipStream_t stream, int keep_y)
{
    if (logDY != 7 && logDY != 8) return hipErrorInvalidValue;
    // keep_y: plain instead of streaming stores of y, for a consumer that reads it at once (a template parameter of the kernels)
    if (N % 128 == 0)
        return keep_y ? launch_wide_t<128, true>(logDY, S, N, K, x, W, y, alpha, stream) : launch_wide_t<128, false>(logDY, S, N, K, x, W, y, alpha, stream);
    return keep_y ? launch_wide_t<64, true>(logDY, S, N, K, x, W, y, alpha, stream) : launch_wide_t<64, false>(logDY, S, N, K, x, W, y, alpha, stream);
}

}  // namespace tfno
