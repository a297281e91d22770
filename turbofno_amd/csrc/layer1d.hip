// Fused 1D spectral layer: forward FFT along DY -> keep 64 modes -> complex GEMM over the channel
// dimension -> zero-pad -> backward FFT, in ONE kernel with no HBM round trip in between.
//
// Replaces fused_fft_cgemm_ifft_{7,8} of the reference
// (fusion_variants/1D_D_exp_fused_fft_cgemm_ifft/fused_fft_cgemm_ifft_7.cuh:9-222): same operands
//   x[K][S][DY]  (signal (k,s) at (k*S+s)*DY),  W[k + n*K],  y[N][S][DY],  M = 64*S,
// the same (S, N/64) blocks (as a 1D grid in an XCD-aware order), block 256, and the same "block traverses K" schedule, re-derived for wave64:
//   * an L = DY/16 lane group owns one signal; a 256-thread block transforms 256/L channels at once
//     (the reference does 8), so the K loop advances in chunks of 16 (DY=256) or 32 (DY=128) channels;
//   * the thread that accumulates C[m][n] is the thread that later needs it for the backward
//     transform, so the GEMM result never passes through LDS (the reference stages it in 8 rounds,
//     fused_fft_cgemm_ifft_7.cuh:203-218);
//   * exchange buffers are padded (row pitch 17 complex) for the 64-bank LDS of CDNA4.
#include "group_fft.h"
#include "kernels.h"

namespace tfno {

// FUSE_FWD: the A operand is produced by forward transforms of x (variants B and D); otherwise it is read from
//           the column-major matrix A[m + k*M] (variant C).
// FUSE_INV: the product goes straight into zero-padded backward transforms (variants C and D); otherwise it is
//           stored as C[m + n*M] = alpha*A*W + beta*C (variant B).
template <int LOGDY, bool FUSE_FWD, bool FUSE_INV, bool KEEP = false>
__global__ __launch_bounds__(256) void fused_fft_cgemm_ifft_kernel(int S, int N, int K, const float2* __restrict__ x,
                                                                   const float2* __restrict__ W, float2* __restrict__ y,
                                                                   float2 alpha, float2 beta)
{
    using G = Geo1D<LOGDY>;
    constexpr int DY = G::DY, L = G::L, GROUPS = G::GROUPS, MM = G::MM, NN = G::NN;
    extern __shared__ float2 lds[];
    float2* sA = lds;                                  // [GROUPS][64]   truncated spectra of the K chunk
    float2* sW = sA + GROUPS * G::SA_PITCH;            // [GROUPS][64]   W chunk, sW[kk][n]
    float2* exch_all = sW + GROUPS * G::SW_PITCH;

    const int tid = threadIdx.x;
    const int g = tid / L, t = tid % L;
    long s;
    int ntile;
    decode_block_1d(S, N / 64, 1 << LOGDY, !KEEP, s, ntile);
    const int n0 = ntile * 64;
    const long M = 64L * S;
    // signals of 128 samples are transformed in pairs by 16-lane groups (128-byte accesses): lane t16 of pair g/2 holds
    // samples t16 + 16 i of both signals, and ends up with the modes an 8-lane group would give lane (g, t)
    constexpr bool PAIR = LOGDY == 7;
    const int t16 = tid % 16, gpair = (tid / 16) * 2;
    float2* exch = PAIR ? exch_all + (tid / 16) * (2 * G::EXCH) : exch_all + g * G::EXCH;

    cpx tw[16];
    load_lane_twiddles<LOGDY>(PAIR ? t16 : t, tw);

    cpx acc[MM][NN];
#pragma unroll
    for (int a = 0; a < MM; ++a)
#pragma unroll
        for (int b = 0; b < NN; ++b) acc[a][b] = make_float2(0.f, 0.f);

    for (int kc = 0; kc < K; kc += GROUPS) {
        if constexpr (FUSE_FWD) {
            const int k = kc + g;
            cpx out[MM];
            if (k < K) {
                cpx v[16];
                if constexpr (PAIR) {
                    const float2* src = x + ((long)(kc + gpair) * S + s) * DY + t16;
#pragma unroll
                    for (int i = 0; i < 8; ++i) { v[i] = src[16 * i]; v[8 + i] = src[(long)S * DY + 16 * i]; }
                    pair128_forward(v, tw, exch, t16, out);
                } else {
                    const float2* src = x + ((long)k * S + s) * DY + t;
#pragma unroll
                    for (int i = 0; i < 16; ++i) v[i] = src[L * i];
                    group_forward<LOGDY>(v, tw, exch, t, out);
                }
            } else {
#pragma unroll
                for (int a = 0; a < MM; ++a) out[a] = make_float2(0.f, 0.f);
            }
#pragma unroll
            for (int a = 0; a < MM; ++a) sA[g * G::SA_PITCH + (PAIR ? t + L * a : forward_mode_of_lane<LOGDY>(t, a))] = out[a];
        } else {
            // A tile of the chunk: 64 contiguous rows (this block's signal) of GROUPS columns
#pragma unroll
            for (int j = 0; j < (GROUPS * 64) / 256; ++j) {
                const int idx = tid + 256 * j;
                const int mloc = idx % 64, kk = idx / 64;
                sA[kk * G::SA_PITCH + mloc] =
                    (kc + kk < K) ? x[s * 64 + mloc + (long)(kc + kk) * M] : make_float2(0.f, 0.f);
            }
        }
        // W chunk: GROUPS x 64 elements, consecutive threads read consecutive k (contiguous in memory)
#pragma unroll
        for (int j = 0; j < (GROUPS * 64) / 256; ++j) {
            int idx = tid + 256 * j;
            int kk = idx % GROUPS, n = idx / GROUPS;
            float2 w = make_float2(0.f, 0.f);
            if (kc + kk < K) w = W[(kc + kk) + (long)(n0 + n) * K];
            sW[kk * G::SW_PITCH + n] = w;
        }
        __syncthreads();
#pragma unroll 4
        for (int kk = 0; kk < GROUPS; ++kk) {
            cpx a[MM], b[NN];
#pragma unroll
            for (int i = 0; i < MM; ++i) a[i] = sA[kk * G::SA_PITCH + t + L * i];
#pragma unroll
            for (int j = 0; j < NN; ++j) b[j] = sW[kk * G::SW_PITCH + g + GROUPS * j];
#pragma unroll
            for (int i = 0; i < MM; ++i)
#pragma unroll
                for (int j = 0; j < NN; ++j) cfma(acc[i][j], a[i], b[j]);
        }
        __syncthreads();
    }

#pragma unroll
    for (int j = 0; j < NN; ++j) {
        const int n = n0 + g + GROUPS * j;
        if constexpr (FUSE_INV) {
            cpx c[MM], yv[16];
#pragma unroll
            for (int i = 0; i < MM; ++i) c[i] = cmul(acc[i][j], alpha);
            if constexpr (PAIR) {
                pair128_backward(c, tw, exch, t16, yv);
                float2* dst = y + ((long)(n0 + gpair + GROUPS * j) * S + s) * DY + t16;
                store_pair16<KEEP>(dst, (long)S * DY, yv);
            } else {
                group_backward<LOGDY>(c, tw, exch, t, yv);
                float2* dst = y + ((long)n * S + s) * DY + t;
                store_row16<L, KEEP>(dst, yv);
            }
        } else {
            float2* dst = y + s * 64 + t + (long)n * M;          // C[m + n*M], m = s*64 + t + L*i
#pragma unroll
            for (int i = 0; i < MM; ++i) {
                cpx r = cmul(acc[i][j], alpha);
                if (beta.x != 0.f || beta.y != 0.f) r = cadd(r, cmul(dst[L * i], beta));
                dst[L * i] = r;
            }
        }
    }
}

// Fused 1D layer with the contraction on the fp32 matrix cores, for channel counts where the GEMM dominates the
// arithmetic (K >= one chunk). Same operands, grid (S, N/64) and block-traverses-K schedule as the kernel above;
// 512 threads = 8 waves:
//   * a chunk is KC = 512/L channels (32 for DY=256, 64 for DY=128): every L-lane group transforms one channel and
//     leaves its 64 modes in sA[k][m]; two chunks of loads are in flight per group (a buffer is refilled as soon as the
//     first pass has consumed it), so they travel under the exchanges, the W tile builds and the matrix work;
//   * C'[n'][m] += W'[n'][k'] A'[k'][m] is the 4-real form of the complex product on v_mfma_f32_16x16x4_f32:
//     n' = (n, re|im) 128 rows, m 64 columns = 8 x 4 tiles, four per wave (one m tile, four n' tiles), so one read of
//     A from LDS feeds eight matrix instructions. W' (alpha folded in) uses the conflict-free LDS order kWGroup / kWHalf;
//     sA has a pitch of 80 complex so that the two k rows a half wave reads fall on disjoint banks;
//   * the product goes through LDS once (sC, pitch 72) to reach the lane groups that run the zero-padded backward
//     transforms and store y.
// sA aliases the exchange regions of the lane groups (the transforms of a chunk are complete before sA is written),
// sC aliases the W' tile.
typedef float floatx4_1d __attribute__((ext_vector_type(4)));

// NT_ = output channels per block: 64, or 32 to spread a small grid over twice as many CUs (DY = 256, 512 threads).
template <int LOGDY, int THREADS_, int NT_ = 64> struct GeoMfma1D {
    static constexpr int L = Geo1D<LOGDY>::L, MM = 64 / L;
    static constexpr int THREADS = THREADS_;                  // 512: one block per CU; 256: two (LDS 72 KiB each)
    static constexpr int NT = NT_;
    static constexpr int NTW = (NT / 2) / (THREADS / 64);     // 16x16 tiles per wave: one m tile x NTW n' tiles
    static constexpr int KC = THREADS / L;                    // channels per chunk = lane groups per block
    // compact: sC shares the exchange regions too and the twiddles move to LDS: 53 KiB and 168 registers, three blocks
    // per CU. Only for DY = 256: at DY = 128 (8 modes per lane) the register limit costs more in spills than it gains.
    static constexpr bool COMPACT = THREADS_ == 256 && LOGDY == 8;
    static constexpr int PA = 80, PC = COMPACT ? 66 : 72;     // pitches (complex) of sA and sC
    static constexpr int EXCH = L * 17;
    static constexpr int REGION0 = KC * EXCH > KC * PA ? KC * EXCH : KC * PA;              // exchange | sA
    static constexpr int WTILE = (KC / 4) * kWGroup / 2;                                   // W' tile in complex units
    static constexpr int REGION1 = COMPACT ? WTILE : (WTILE > NT * PC ? WTILE : NT * PC);  // W' | sC   (complex)
    static_assert(!COMPACT || NT * PC <= REGION0, "sC must fit the exchange regions");
    static_assert(NT == 64 || (NT == 32 && THREADS_ == 512), "32-channel tiles: 512 threads");
    static constexpr int PASSES = (NT + KC - 1) / KC;         // backward passes; the last may use only NT % KC lane groups
    static constexpr int TWTAB = COMPACT ? kTwLdsSize : 0;    // compact: twiddles in LDS instead of 30 registers
    static constexpr int DEPTH = COMPACT ? 1 : 2;             // chunks of loads in flight per lane group
    static constexpr size_t LDS_BYTES = sizeof(float2) * (size_t)(REGION0 + REGION1 + TWTAB);
};

template <int LOGDY, int THREADS, int NT, bool KEEP = false>
__global__ __launch_bounds__(THREADS, (THREADS == 256 && LOGDY == 8) ? 3 : 1) void fused_fft_mfma_ifft_kernel(int S, int N, int K, const float2* __restrict__ x,
                                                                      const float2* __restrict__ W, float2* __restrict__ y,
                                                                      float2 alpha)
{
    using G = GeoMfma1D<LOGDY, THREADS, NT>;
    constexpr int NTW = G::NTW;
    constexpr int DY = 1 << LOGDY, L = G::L, MM = G::MM, KC = G::KC, PA = G::PA, PC = G::PC;
    extern __shared__ float2 lds[];
    float2* sA = lds;                                          // [KC][PA]; aliases the exchange regions
    float* sW = reinterpret_cast<float*>(lds + G::REGION0);    // W' tile, layout of kWGroup / kWHalf
    float2* sC = G::COMPACT ? lds : lds + G::REGION0;          // [64][PC]; aliases sW (or sA) after the K loop

    const int tid = threadIdx.x;
    const int g = tid / L, t = tid % L;                        // transform role: lane group = channel of the chunk
    const int wave = tid >> 6, lane = tid & 63, col = lane & 15, kq = lane >> 4;   // matrix role
    const int mt = wave & 3, nt0 = (wave >> 2) * NTW;          // m tile, first of the wave's NTW n' tiles
    long s;
    int ntile;
    decode_block_1d(S, N / NT, 1 << LOGDY, !KEEP, s, ntile);
    const int n0 = ntile * NT;
    // DY = 128: signals are transformed in pairs by 16-lane groups (see the SIMT kernel); COMPACT never applies there
    constexpr bool PAIR = LOGDY == 7;
    const int t16 = tid % 16, gpair = (tid / 16) * 2;
    float2* exch = PAIR ? lds + (tid / 16) * (2 * G::EXCH) : lds + g * G::EXCH;

    cpx tw[16];
    const float2* twrow = lds + G::REGION0 + G::REGION1 + t * kTwLdsPitch;
    if constexpr (G::COMPACT) {
        fill_lds_twiddles<LOGDY>(lds + G::REGION0 + G::REGION1, tid, THREADS);
        __syncthreads();
    } else {
        load_lane_twiddles<LOGDY>(PAIR ? t16 : t, tw);
    }

    floatx4_1d acc[NTW];
#pragma unroll
    for (int i = 0; i < NTW; ++i) acc[i] = floatx4_1d{ 0.f, 0.f, 0.f, 0.f };

    // loads of this lane group's channel(s) of the chunk that starts at channel kc
    auto issue = [&](cpx (&dst)[16], int kc) {
        if constexpr (PAIR) {
            const float2* src = x + ((long)(kc + gpair) * S + s) * DY + t16;
#pragma unroll
            for (int i = 0; i < 8; ++i) { dst[i] = src[16 * i]; dst[8 + i] = src[(long)S * DY + 16 * i]; }
        } else {
            const float2* src = x + ((long)(kc + g) * S + s) * DY + t;
#pragma unroll
            for (int i = 0; i < 16; ++i) dst[i] = src[L * i];
        }
    };
    // two chunks of loads in flight per lane group: buffer b receives chunk c + 2 as soon as chunk c has left it
    cpx v0[16], v1[16];
    if (g < K) issue(v0, 0);
    if (G::DEPTH == 2 && KC + g < K) issue(v1, KC);

    auto chunk = [&](cpx (&v)[16], int kc) {
        const int kn = (K - kc) < KC ? (K - kc) : KC;          // multiple of 8 (caller contract)
        // W chunk: lanes run along k, the contiguous direction of W[k + n*K]
        constexpr int WPT = KC * NT / G::THREADS;
        float2 wv[WPT];
#pragma unroll
        for (int u = 0; u < WPT; ++u) {
            const int idx = tid + u * G::THREADS;
            const int k = idx % KC, n = idx / KC;
            wv[u] = (k < kn) ? W[(kc + k) + (long)(n0 + n) * K] : make_float2(0.f, 0.f);
        }
        cpx out[MM];
        if (g < kn) {
            if constexpr (PAIR) {
                cpx w[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) w[i] = v[i];
                if (kc + G::DEPTH * KC + g < K) issue(v, kc + G::DEPTH * KC);
                pair128_forward(w, tw, exch, t16, out);
            } else {
                cpx gg[16];
                if constexpr (G::COMPACT) fwd_pass1_lds(v, twrow, gg);
                else fwd_pass1(v, tw, gg);
                if (kc + G::DEPTH * KC + g < K) issue(v, kc + G::DEPTH * KC);    // the chunk DEPTH chunks ahead
                group_forward_finish<LOGDY>(gg, exch, t, out);
            }
        }
        __syncthreads();                                       // all exchanges done: sA may overwrite them
        if (g < kn) {
#pragma unroll
            for (int a = 0; a < MM; ++a) sA[g * PA + (PAIR ? t + L * a : forward_mode_of_lane<LOGDY>(t, a))] = out[a];
        }
#pragma unroll
        for (int u = 0; u < WPT; ++u) {
            const int idx = tid + u * G::THREADS;
            const int k = idx % KC, n = idx / KC;
            const float2 w = make_float2(wv[u].x * alpha.x - wv[u].y * alpha.y, wv[u].x * alpha.y + wv[u].y * alpha.x);
            float* dstw = &sW[(k >> 2) * kWGroup + ((k & 3) >> 1) * kWHalf + (2 * n) * 4 + (k & 1) * 2];
            *reinterpret_cast<float2*>(dstw) = make_float2(w.x, -w.y);
            *reinterpret_cast<float2*>(dstw + 4) = make_float2(w.y, w.x);
        }
        __syncthreads();
        const float2* arow = sA + kq * PA + mt * 16 + col;
        const float* wrow = sW + (kq >> 1) * kWHalf + (nt0 * 16 + col) * 4 + (kq & 1) * 2;
        for (int kg = 0; kg < kn / 4; ++kg) {
            const float2 b = arow[kg * 4 * PA];
#pragma unroll
            for (int i = 0; i < NTW; ++i) {
                const float2 a = *reinterpret_cast<const float2*>(wrow + kg * kWGroup + i * 64);
                acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, acc[i], 0, 0, 0);
                acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, acc[i], 0, 0, 0);
            }
        }
        __syncthreads();                                       // sA / sW are free again (next chunk, or sC below)
    };
    for (int kc = 0; kc < K; kc += G::DEPTH * KC) {
        chunk(v0, kc);
        if (G::DEPTH == 2 && kc + KC < K) chunk(v1, kc + KC);
    }

    // D[row = 4 kq + v][col] of tile i: n' = 16 (nt0 + i) + 4 kq + v = 2 n + c'  ->  n = 8 (nt0 + i) + 2 kq + (v >> 1)
#pragma unroll
    for (int i = 0; i < NTW; ++i) {
        const int n = 8 * (nt0 + i) + 2 * kq;
        sC[n * PC + mt * 16 + col] = make_float2(acc[i][0], acc[i][1]);
        sC[(n + 1) * PC + mt * 16 + col] = make_float2(acc[i][2], acc[i][3]);
    }
    __syncthreads();
    // every pass takes its modes before the first backward transform: in the compact layout the exchange regions
    // overlay sC
    cpx c[G::PASSES][MM];
#pragma unroll
    for (int pass = 0; pass < G::PASSES; ++pass)
#pragma unroll
        for (int a = 0; a < MM; ++a) c[pass][a] = (g + KC * pass < NT) ? sC[(g + KC * pass) * PC + t + L * a] : make_float2(0.f, 0.f);
    if constexpr (G::COMPACT) __syncthreads();
#pragma unroll
    for (int pass = 0; pass < G::PASSES; ++pass) {
        const int n = g + KC * pass;
        if (n >= NT) break;                                    // whole waves (NT and KC are multiples of 32 channels)
        cpx yv[16];
        if constexpr (PAIR) {
            pair128_backward(c[pass], tw, exch, t16, yv);
            float2* dst = y + ((long)(n0 + gpair + KC * pass) * S + s) * DY + t16;
            store_pair16<KEEP>(dst, (long)S * DY, yv);
        } else {
            if constexpr (G::COMPACT) group_backward_lds<LOGDY>(c[pass], twrow, exch, t, yv);
            else group_backward<LOGDY>(c[pass], tw, exch, t, yv);
            float2* dst = y + ((long)(n0 + n) * S + s) * DY + t;
            store_row16<L, KEEP>(dst, yv);
        }
    }
}

// Fused 1D layer for large grids, DY = 128 / 256: ONE WAVEFRONT per (signal set, 64 output channels), no block barrier
// and no staging of operands through LDS. The register layouts of the transforms and of v_mfma_f32_16x16x4_f32 coincide:
//   * DY = 256: the four 16-lane groups of a wave transform four channels k = kc + g at a time and lane (g, t) ends up
//     with modes t + 16 a, a < 4, of channel g: exactly the B operand (k = lane / 16, column = lane % 16) of the four
//     m tiles a;
//   * the A operand row n' = 16 nt + t, k = g is one element of W (times alpha, as (re, -im) or (im, re)), read
//     straight from global memory (W is a few KiB and stays in the vector cache);
//   * the accumulators D[row = 4 g + v][column = t] of tile (nt, a) hold, for j = 0, 1, the complex value
//     (v = 2 j, 2 j + 1) of output channel n = 8 nt + 2 g + j at mode t + 16 a: the input layout of the zero-padded
//     backward transform of channel n by lane group g;
//   * DY = 128: a lane group transforms two channels kc + 2 g + h at a time (lane t = r + 8 h finishes channel h with
//     modes r + 8 c, c < 8); one exchange between lanes t and t ^ 8 (a row rotation, no LDS) turns that into modes
//     t + 16 a of each of the two channels, i.e. two B operands, and the same exchange leads from the accumulators to
//     the paired backward transform of output channels 8 nt + 2 g and 8 nt + 2 g + 1.
// 32 accumulator tiles (128 registers) per wave, two waves per SIMD; the only LDS traffic left is the exchange inside
// the transforms. The loads of the next channels are issued as soon as the first pass has consumed the current ones
// and travel under the exchange, the second pass and the matrix instructions (64 per four channels).
TFNO_DEV float rotate8(float v)        // value of lane t ^ 8 of the same 16-lane row
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128 /* row_ror:8 */, 0xf, 0xf, false));
}
TFNO_DEV cpx rotate8(cpx v) { return make_float2(rotate8(v.x), rotate8(v.y)); }

template <int LOGDY, bool KEEP = false>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2, 2))) void fused_fft_mfma_ifft_wave_kernel(
    int S, int N, int K, const float2* __restrict__ x, const float2* __restrict__ W, float2* __restrict__ y, float2 alpha)
{
    constexpr int DY = 1 << LOGDY, EXCH = 16 * 17;
    constexpr bool PAIR = LOGDY == 7;
    constexpr int CH = PAIR ? 8 : 4;                              // channels per round
    constexpr int REGIONS = PAIR ? 4 : 8;                         // DY = 256: a second set for the paired backward transforms
    __shared__ float2 lds[REGIONS * EXCH + kTwLdsSize];
    const int lane = threadIdx.x, g = lane >> 4, t = lane & 15;
    float2* exch = lds + g * EXCH;
    float2* exch1 = exch + (PAIR ? 0 : 4 * EXCH);                 // second region: two backward transforms in flight
    float2* twtab = lds + REGIONS * EXCH;
    fill_lds_twiddles<LOGDY>(twtab, lane, 64);
    const float2* twrow = twtab + t * kTwLdsPitch;
    __syncthreads();
    long s;
    int ntile;
    decode_block_1d(S, N / 64, 1 << LOGDY, !KEEP, s, ntile);
    const int n0 = ntile * 64;
    const bool upper = t >> 3, odd = t & 1;

    floatx4_1d acc[8][4];
#pragma unroll
    for (int nt = 0; nt < 8; ++nt)
#pragma unroll
        for (int a = 0; a < 4; ++a) acc[nt][a] = floatx4_1d{ 0.f, 0.f, 0.f, 0.f };

    // lane (g, t): samples t + 16 i of channel kc + g (DY = 256) or of channels kc + 2 g, kc + 2 g + 1 (DY = 128)
    const float2* src = x + ((long)(PAIR ? 2 * g : g) * S + s) * DY + t;
    const float2* wsrc = W + (PAIR ? 2 * g : g) + (long)(n0 + (t >> 1)) * K;   // W[k][n = n0 + 8 nt + t / 2]
    auto issue = [&](cpx (&dst)[16]) {
        if constexpr (PAIR) {
#pragma unroll
            for (int i = 0; i < 8; ++i) { dst[i] = src[16 * i]; dst[8 + i] = src[(long)S * DY + 16 * i]; }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) dst[i] = src[16 * i];
        }
    };
    // one complex product row: acc += W'(row n', k) x B(k, column), W' = alpha W as (re, -im) / (im, re) by row parity
    auto contract = [&](floatx4_1d (&d)[4], float2 wk, const cpx (&b)[4]) {
        const float2 w = make_float2(wk.x * alpha.x - wk.y * alpha.y, wk.x * alpha.y + wk.y * alpha.x);
        const float ax = odd ? w.y : w.x, ay = odd ? w.x : -w.y;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            d[a] = __builtin_amdgcn_mfma_f32_16x16x4f32(ax, b[a].x, d[a], 0, 0, 0);
            d[a] = __builtin_amdgcn_mfma_f32_16x16x4f32(ay, b[a].y, d[a], 0, 0, 0);
        }
    };
    cpx v[16];
    issue(v);
    for (int kc = 0; kc < K; kc += CH) {                          // K is a multiple of 8 (caller contract)
        float2 wv[8], wv1[8];
#pragma unroll
        for (int nt = 0; nt < 8; ++nt) {
            wv[nt] = wsrc[kc + (long)(8 * nt) * K];
            if constexpr (PAIR) wv1[nt] = wsrc[kc + 1 + (long)(8 * nt) * K];
        }
        if constexpr (!PAIR) {
            cpx gg[16], out[4];
            fwd_pass1_lds(v, twrow, gg);
            if (kc + CH < K) { src += (long)CH * S * DY; issue(v); }
            group_forward_finish<8>(gg, exch, t, out);
#pragma unroll
            for (int nt = 0; nt < 8; ++nt) contract(acc[nt], wv[nt], out);
        } else {
            cpx gg[16], out[8], b8[8];
            {
                cpx a8[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) { a8[i] = v[i]; b8[i] = v[8 + i]; }
                fft8<-1>(a8);
                fft8<-1>(b8);
#pragma unroll
                for (int r = 0; r < 8; ++r) gg[r] = a8[r];
            }
            if (kc + CH < K) { src += (long)CH * S * DY; issue(v); }
            gg[8] = b8[0];
#pragma unroll
            for (int r = 1; r < 8; ++r) {
                const cpx w = twrow[r];
                gg[r] = cmul(gg[r], w);
                gg[8 + r] = cmul(b8[r], w);
            }
            rows128_forward_finish(gg, exch, t, out);             // out[c] = mode (t & 7) + 8 c of channel t >> 3
            // lanes t < 8 keep the even c of their channel and take the even c of the other one; lanes t >= 8 the odd c
            cpx b0[4], b1[4];
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const cpx got = rotate8(upper ? out[2 * a] : out[2 * a + 1]);
                b0[a] = upper ? got : out[2 * a];                 // channel kc + 2 g,     mode t + 16 a
                b1[a] = upper ? out[2 * a + 1] : got;             // channel kc + 2 g + 1, mode t + 16 a
            }
#pragma unroll
            for (int nt = 0; nt < 8; ++nt) {
                contract(acc[nt], wv[nt], b0);
                contract(acc[nt], wv1[nt], b1);
            }
        }
    }
    // backward: the two output channels (j = 0, 1) a lane group owns per n tile are transformed together
#pragma unroll
    for (int nt = 0; nt < 8; ++nt) {
        cpx c0[4], c1[4], y0[16], y1[16];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            c0[a] = make_float2(acc[nt][a][0], acc[nt][a][1]);   // channel 8 nt + 2 g,     mode t + 16 a
            c1[a] = make_float2(acc[nt][a][2], acc[nt][a][3]);   // channel 8 nt + 2 g + 1, mode t + 16 a
        }
        float2* dst = y + ((long)(n0 + 8 * nt + 2 * g) * S + s) * DY + t;
        if constexpr (!PAIR) {
            // each through its own exchange region, so that the LDS round trips of one overlap the arithmetic of the other
            cpx h0[16], h1[16], e0[16], e1[16];
            dft16_pad4<+1>(c0, h0);
            dft16_pad4<+1>(c1, h1);
            wave_lds_fence();
#pragma unroll
            for (int tt = 0; tt < 16; ++tt) { exch[tt * 17 + t] = h0[tt]; exch1[tt * 17 + t] = h1[tt]; }
            wave_lds_fence();
#pragma unroll
            for (int r = 0; r < 16; ++r) { e0[r] = exch[t * 17 + r]; e1[r] = exch1[t * 17 + r]; }
            inv_pass2_lds(e0, twrow, y0);
            inv_pass2_lds(e1, twrow, y1);
            store_row16<16, KEEP>(dst, y0);
            store_row16<16, KEEP>(dst + (long)S * DY, y1);
        } else {
            // lane t = r + 8 h finishes channel h: modes r + 8 c; even c come from lanes t < 8, odd c from lanes t >= 8
            cpx c8[8];
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const cpx got = rotate8(upper ? c0[a] : c1[a]);
                c8[2 * a] = upper ? got : c0[a];
                c8[2 * a + 1] = upper ? c1[a] : got;
            }
            rows128_backward(c8, twrow, exch, t, y0);
            store_pair16<KEEP>(dst, (long)S * DY, y0);
        }
    }
}

// Fused 1D layer for small grids (every block has a CU to itself), DY = 256: the eight waves of a block share ONE
// item (signal set, 32 output channels) and split its K input channels. Operands as in the one-wavefront kernel above:
// wave w transforms channels 32 r + 4 w + g in round r and multiplies them straight out of its registers into its own
// partial accumulators (4 n' tiles x 4 m tiles), so the K loop has no barrier and stages nothing through LDS. The
// eight partial products meet in LDS once (sP[w][n][m], pitch 72 complex: conflict-free b64 stores), every lane group
// sums the eight partials of one output channel and runs its backward transform. The chain of latencies of an item
// is K / 32 rounds + one reduction + one backward pass, against three barriers and two tile builds per 32 channels
// in the kernel that shares the spectra through LDS.
constexpr int SPLIT_NT = 32, SPLIT_PP = 72;
constexpr size_t SPLIT_LDS = sizeof(float2) * 8 * SPLIT_NT * SPLIT_PP;       // 147,456 B; covers the 32 exchange regions

__global__ __launch_bounds__(512) void fused_fft_mfma_ifft_split_kernel(int S, int N, int K, const float2* __restrict__ x,
                                                                        const float2* __restrict__ W, float2* __restrict__ y,
                                                                        float2 alpha)
{
    constexpr int DY = 256, EXCH = 16 * 17;
    extern __shared__ float2 lds[];
    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, t = lane & 15;
    float2* exch = lds + (4 * w + g) * EXCH;                      // the partials overlay these after the K loop
    long s;
    int ntile;
    decode_block_1d(S, N / SPLIT_NT, 256, true, s, ntile);
    const int n0 = ntile * SPLIT_NT;
    const bool odd = t & 1;
    cpx tw[16];
    load_lane_twiddles<8>(t, tw);

    floatx4_1d acc[4][4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int a = 0; a < 4; ++a) acc[nt][a] = floatx4_1d{ 0.f, 0.f, 0.f, 0.f };

    // K is a multiple of 8 and a wave covers four consecutive channels: a wave is either fully inside K or idle
    const int k0 = 4 * w + g;
    const float2* src = x + ((long)k0 * S + s) * DY + t;
    const float2* wsrc = W + k0 + (long)(n0 + (t >> 1)) * K;      // W[k][n = n0 + 8 nt + t / 2]
    auto issue = [&](cpx (&dst)[16], int kc) {                    // samples t + 16 i of channel kc + k0
        const float2* p = src + (long)kc * S * DY;
#pragma unroll
        for (int i = 0; i < 16; ++i) dst[i] = p[16 * i];
    };
    // the buffer is refilled as soon as the first pass has consumed it (a second buffer, two rounds ahead, was
    // measured slower: a round is bound by its arithmetic, not by the latency of its loads)
    auto round = [&](cpx (&v)[16], int kc) {
        float2 wv[4];
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) wv[nt] = wsrc[kc + (long)(8 * nt) * K];
        cpx gg[16], out[4];
        fwd_pass1(v, tw, gg);
        if (kc + 32 + 4 * w < K) issue(v, kc + 32);
        group_forward_finish<8>(gg, exch, t, out);
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
            const float2 wa = make_float2(wv[nt].x * alpha.x - wv[nt].y * alpha.y, wv[nt].x * alpha.y + wv[nt].y * alpha.x);
            const float ax = odd ? wa.y : wa.x, ay = odd ? wa.x : -wa.y;
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                acc[nt][a] = __builtin_amdgcn_mfma_f32_16x16x4f32(ax, out[a].x, acc[nt][a], 0, 0, 0);
                acc[nt][a] = __builtin_amdgcn_mfma_f32_16x16x4f32(ay, out[a].y, acc[nt][a], 0, 0, 0);
            }
        }
    };
    cpx v[16];
    if (4 * w < K) issue(v, 0);
    for (int kc = 0; kc + 4 * w < K; kc += 32) round(v, kc);
    __syncthreads();                                              // every wave is done with its exchange regions
    // D[row = 4 g + v][column = t] of tile (nt, a): channel n = 8 nt + 2 g + (v >> 1), re | im = v & 1, mode t + 16 a
    float2* sP = lds + (long)w * SPLIT_NT * SPLIT_PP;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            sP[(8 * nt + 2 * g) * SPLIT_PP + t + 16 * a] = make_float2(acc[nt][a][0], acc[nt][a][1]);
            sP[(8 * nt + 2 * g + 1) * SPLIT_PP + t + 16 * a] = make_float2(acc[nt][a][2], acc[nt][a][3]);
        }
    __syncthreads();
    // lane group (w, g) owns output channel n = 4 w + g: sum of the eight partials, modes t + 16 a
    const int n = 4 * w + g;
    cpx c[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        cpx sum = lds[n * SPLIT_PP + t + 16 * a];
#pragma unroll
        for (int ww = 1; ww < 8; ++ww) sum = cadd(sum, lds[(ww * SPLIT_NT + n) * SPLIT_PP + t + 16 * a]);
        c[a] = sum;
    }
    __syncthreads();                                              // the partials are consumed: exchange regions again
    cpx yv[16];
    group_backward<8>(c, tw, exch, t, yv);
    float2* dst = y + ((long)(n0 + n) * S + s) * DY + t;
#pragma unroll
    for (int i = 0; i < 16; ++i) store_streaming(dst + 16 * i, yv[i]);
}

// Stand-alone truncated forward / zero-padded backward transforms of contiguous signals (variants A, B, C):
//   fft_stride_DY : in[nsig][DY] -> out[nsig][64]      ifft_stride_DY : in[nsig][64] -> out[nsig][DY]
// Replace fft_N_stride_DY / ifft_N_stride_DY of the missing TurboFFT submodule (launched at
// fusion_variants/1D_A_exp_fft+cgemm+ifft/fused.cu:195,203). One L-lane group per signal, 256/L signals per block.
template <int LOGDY, bool INVERSE>
__global__ __launch_bounds__(256) void stride_DY_kernel(const float2* __restrict__ in, float2* __restrict__ out, long nsig)
{
    using G = Geo1D<LOGDY>;
    constexpr int DY = G::DY, L = G::L, GROUPS = G::GROUPS, MM = G::MM;
    extern __shared__ float2 lds[];
    const int tid = threadIdx.x, g = tid / L, t = tid % L;
    const long sig = (long)blockIdx.x * GROUPS + g;
    cpx tw[16];
    if constexpr (LOGDY == 7) {
        // signals of 128 samples go in pairs through 16-lane groups (128-byte accesses); lane (g, t) still ends up with /
        // starts from the modes t + 8 a of signal g. All 16 lanes take part for either signal, so a pair with one
        // signal beyond nsig loads zeros for it and skips its stores instead of leaving early.
        const int t16 = tid % 16;
        const long sigA = (long)blockIdx.x * GROUPS + (tid / 16) * 2;
        float2* exch = lds + (tid / 16) * (2 * G::EXCH);
        load_lane_twiddles<LOGDY>(t16, tw);
        if (sigA >= nsig) return;                    // whole pair out of range (uniform per 16-lane group)
        const bool hasB = sigA + 1 < nsig;
        if constexpr (!INVERSE) {
            const float2* src = in + sigA * DY + t16;
            cpx v[16], o[MM];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                v[i] = src[16 * i];
                v[8 + i] = hasB ? src[DY + 16 * i] : make_float2(0.f, 0.f);
            }
            pair128_forward(v, tw, exch, t16, o);
            if (sig < nsig) {
                float2* dst = out + sig * 64 + t;
#pragma unroll
                for (int a = 0; a < MM; ++a) dst[L * a] = o[a];
            }
        } else {
            cpx c[MM], yv[16];
#pragma unroll
            for (int a = 0; a < MM; ++a) c[a] = sig < nsig ? in[sig * 64 + t + L * a] : make_float2(0.f, 0.f);
            pair128_backward(c, tw, exch, t16, yv);
            float2* dst = out + sigA * DY + t16;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                store_streaming(dst + 16 * i, yv[i]);
                if (hasB) store_streaming(dst + DY + 16 * i, yv[8 + i]);
            }
        }
        return;
    } else {
    float2* exch = lds + g * G::EXCH;
    load_lane_twiddles<LOGDY>(t, tw);
    if (sig >= nsig) return;
    if constexpr (!INVERSE) {
        const float2* src = in + sig * DY + t;
        cpx v[16], o[MM];
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = src[L * i];
        group_forward<LOGDY>(v, tw, exch, t, o);
        float2* dst = out + sig * 64;
#pragma unroll
        for (int a = 0; a < MM; ++a) dst[forward_mode_of_lane<LOGDY>(t, a)] = o[a];
    } else {
        const float2* src = in + sig * 64 + t;
        cpx c[MM], yv[16];
#pragma unroll
        for (int a = 0; a < MM; ++a) c[a] = src[L * a];
        group_backward<LOGDY>(c, tw, exch, t, yv);
        float2* dst = out + sig * DY + t;
#pragma unroll
        for (int i = 0; i < 16; ++i) store_streaming(dst + L * i, yv[i]);
    }
    }
}

template <int LOGDY, bool FUSE_FWD, bool FUSE_INV, bool KEEP>
static hipError_t launch_fused_1d_k(long S, int N, int K, const float2* x, const float2* W, float2* y, float2 alpha,
                                    float2 beta, hipStream_t stream)
{
    using G = Geo1D<LOGDY>;
    if (S * (N / 64) > 0x7fffffffL) return hipErrorInvalidValue;
    if constexpr (G::LDS_BYTES > 64 * 1024) {          // DY = 128: 32 channels per chunk, 70 KiB
        static std::atomic<unsigned long long> served;
        if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(fused_fft_cgemm_ifft_kernel<LOGDY, FUSE_FWD, FUSE_INV, KEEP>),
                                             G::LDS_BYTES, served);
            e != hipSuccess)
            return e;
    }
    dim3 grid((unsigned)(S * (N / 64)), 1, 1), block(256, 1, 1);
    hipLaunchKernelGGL((fused_fft_cgemm_ifft_kernel<LOGDY, FUSE_FWD, FUSE_INV, KEEP>), grid, block, G::LDS_BYTES, stream, (int)S,
                       N, K, x, W, y, alpha, beta);
    return hipGetLastError();
}

// keep_y: the output is read again at once (Y stage of the three-kernel 2D pipeline): plain instead of streaming stores,
// as a template parameter of the kernels - a run-time branch around the stores cost the 1D layer up to 20 %
template <int LOGDY, bool FUSE_FWD, bool FUSE_INV>
static hipError_t launch_fused_1d(long S, int N, int K, const float2* x, const float2* W, float2* y, float2 alpha,
                                  float2 beta, hipStream_t stream, int keep_y = 0)
{
    if constexpr (FUSE_FWD && FUSE_INV) {
        if (keep_y) return launch_fused_1d_k<LOGDY, FUSE_FWD, FUSE_INV, true>(S, N, K, x, W, y, alpha, beta, stream);
    }
    return launch_fused_1d_k<LOGDY, FUSE_FWD, FUSE_INV, false>(S, N, K, x, W, y, alpha, beta, stream);
}

template <bool FUSE_FWD, bool FUSE_INV>
static hipError_t dispatch_fused_1d(int logDY, long S, int N, int K, const float2* x, const float2* W, float2* y,
                                    float2 alpha, float2 beta, hipStream_t stream, int keep_y = 0)
{
    switch (logDY) {
    case 7: return launch_fused_1d<7, FUSE_FWD, FUSE_INV>(S, N, K, x, W, y, alpha, beta, stream, keep_y);
    case 8: return launch_fused_1d<8, FUSE_FWD, FUSE_INV>(S, N, K, x, W, y, alpha, beta, stream, keep_y);
    case 9: return launch_fused_1d<9, FUSE_FWD, FUSE_INV>(S, N, K, x, W, y, alpha, beta, stream, keep_y);
    case 10: return launch_fused_1d<10, FUSE_FWD, FUSE_INV>(S, N, K, x, W, y, alpha, beta, stream, keep_y);
    default: return hipErrorInvalidValue;
    }
}

template <int LOGDY, int THREADS, int NT, bool KEEP>
static hipError_t launch_fused_mfma_k(long S, int N, int K, const float2* x, const float2* W, float2* y, float2 alpha,
                                      hipStream_t stream)
{
    using G = GeoMfma1D<LOGDY, THREADS, NT>;
    static std::atomic<unsigned long long> served;
    if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(fused_fft_mfma_ifft_kernel<LOGDY, THREADS, NT, KEEP>),
                                         G::LDS_BYTES, served);
        e != hipSuccess)
        return e;
    if (S * (N / NT) > 0x7fffffffL) return hipErrorInvalidValue;
    hipLaunchKernelGGL((fused_fft_mfma_ifft_kernel<LOGDY, THREADS, NT, KEEP>), dim3((unsigned)(S * (N / NT))), dim3(THREADS),
                       G::LDS_BYTES, stream, (int)S, N, K, x, W, y, alpha);
    return hipGetLastError();
}
template <int LOGDY, int THREADS, int NT = 64>
static hipError_t launch_fused_mfma(long S, int N, int K, const float2* x, const float2* W, float2* y, float2 alpha,
                                    hipStream_t stream, int keep_y = 0)
{
    return keep_y ? launch_fused_mfma_k<LOGDY, THREADS, NT, true>(S, N, K, x, W, y, alpha, stream)
                  : launch_fused_mfma_k<LOGDY, THREADS, NT, false>(S, N, K, x, W, y, alpha, stream);
}

template <int LOGDY>
static hipError_t launch_fused_wave(long S, int N, int K, const float2* x, const float2* W, float2* y, float2 alpha,
                                    hipStream_t stream, int keep_y = 0)
{
    if (S * (N / 64) > 0x7fffffffL) return hipErrorInvalidValue;
    if (keep_y)
        hipLaunchKernelGGL((fused_fft_mfma_ifft_wave_kernel<LOGDY, true>), dim3((unsigned)(S * (N / 64))), dim3(64), 0, stream, (int)S, N,
                           K, x, W, y, alpha);
    else
        hipLaunchKernelGGL((fused_fft_mfma_ifft_wave_kernel<LOGDY, false>), dim3((unsigned)(S * (N / 64))), dim3(64), 0, stream, (int)S,
                           N, K, x, W, y, alpha);
    return hipGetLastError();
}

// Which fused 1D kernel runs for a problem: pure arithmetic on the sizes, the selector `algo`, the number of compute
// units and whether the stream has an exchange buffer attached (no device call), so that callers and tests can ask.
// algo: 0 = by size, 1 = SIMT kernel, 2 = matrix cores with 512-thread blocks, 3 = matrix cores with 256-thread blocks,
// 4 = as 2 with 32-channel output tiles, 5 = matrix cores, one wavefront per (signal set, output tile),
// 6 = matrix cores, the eight waves of a block split the K channels of one item (DY = 256),
// 7 = matrix cores, a cluster of blocks splits the K channels of one signal set (DY = 256, N = 64 / 128, small grids),
// 8 = matrix cores, 256-thread blocks with tiles of 128 output channels, three real products per complex one (DY = 256)
// The return value uses the same numbers (1 ... 8). A selector value that a kernel is not built for falls back to the
// choice by size.
//
// By size (measured on MI355X):
//  * while every block has a CU to itself: matrix cores, 8 waves per block - the shortest chain of latencies for
//    every K, even K = 8 where most of a chunk is padding;
//  * grids of several items per SIMD: one wavefront per item (no barriers, nothing staged through LDS). At DY = 128
//    it is ahead from two (K <= 16), four (K < 128) or eight items per CU; at DY = 256, where the block kernels are
//    closer to what the access pattern allows, for K >= 128 (2-8 % from eight items per CU) and, K >= 24, on the
//    very largest grids (4-6 % from 128 items per CU); below that the 256-thread block kernel is level or up to
//    13 % ahead;
//  * otherwise: matrix cores, 256-thread blocks, two or three per CU, for every K - measured 5-27 % ahead of the
//    SIMT kernel on grids of 1 to 12 items per CU also for K < 32, where most of a chunk is padding (lengths
//    512 / 1024: a tie within a few percent for every K, the SIMT kernel stays; on small grids the 512-thread
//    kernel is 30-40 % ahead there too).
int pick_fused_1d_kernel(int logDY, long S, int N, int K, int algo, bool keep_y, long cus, bool exchange_attached)
{
    const bool built = logDY >= 7 && logDY <= 10;
    const bool long_signal = logDY >= 9;            // 512 / 1024: on large grids the block kernels tie with the SIMT kernel
    const long items = S * (N / 64);
    if (algo == 5 && (logDY == 7 || logDY == 8)) return kFused1dWave;
    // N a multiple of 128, DY = 256, K >= 16: blocks with tiles of 128 output channels (every input channel transformed
    // once per signal set, three real products per complex one): 5-20 % ahead of the kernels below on every grid that
    // fills its two slots per CU reasonably evenly (measured from 400 blocks up; with a last round under three quarters
    // full the 64-channel kernels, with their finer blocks, are ahead)
    if (algo == 0 && logDY == 8 && N % 128 == 0 && K >= 16) {
        const long blocks = S * (N / 128), slots = 2L * cus, rounds = (blocks + slots - 1) / slots;
        if (blocks > cus && 4 * blocks >= 3 * rounds * slots) return kFused1dWide;
    }
    // the same at DY = 128 for K >= 64 (3-21 % ahead up to 64 blocks per CU; with fewer channels, or on the very largest
    // grids, the one-wavefront kernel below is level or ahead)
    if (algo == 0 && logDY == 7 && N % 128 == 0 && K >= 64) {
        const long blocks = S * (N / 128), slots = 2L * cus, rounds = (blocks + slots - 1) / slots;
        if (blocks > cus && blocks <= 64L * cus && 4 * blocks >= 3 * rounds * slots) return kFused1dWide;
    }
    // DY = 128, about one wide block per CU (three quarters to all of them), 16 channels or more: 5-32 % ahead of the
    // kernels below, whose blocks are finer than there are CUs to fill
    if (algo == 0 && logDY == 7 && N % 128 == 0 && K >= 16) {
        const long blocks = S * (N / 128);
        if (4 * blocks >= 3L * cus && blocks <= cus) return kFused1dWide;
    }
    // DY = 128 with N not a multiple of 128 (tiles of 64, three real products): one to two blocks per CU, 16 channels or
    // more: 6-22 % ahead; with 128 channels up to four per CU (12 %)
    if (algo == 0 && logDY == 7 && N % 128 != 0 && K >= 16) {
        const long blocks = S * (N / 64);
        if (blocks >= cus && blocks <= (K >= 128 ? 4L : 2L) * cus) return kFused1dWide;
    }
    // DY = 256, N not a multiple of 128, 128 channels or more, up to four blocks of 64-channel tiles per CU: 6-8 % ahead
    if (algo == 0 && logDY == 8 && N % 128 != 0 && K >= 128) {
        const long blocks = S * (N / 64);
        if (blocks > cus && blocks <= 4L * cus) return kFused1dWide;
    }
    if (algo == 0 && logDY == 7 && items >= (K <= 16 ? 2 : (K < 128 ? 4 : 8)) * cus) return kFused1dWave;
    if (algo == 0 && logDY == 8 && (K >= 128 ? items >= 8L * cus : (K >= 24 && items >= 128L * cus))) return kFused1dWave;
    // small grids, 64 channels or more, N = 64 / 128: a cluster of blocks per signal set, no forward transform twice.
    // Only for streams that have an exchange buffer attached; without one the kernels below take over.
    if (algo == 7 || (algo == 0 && logDY == 8 && K >= 64)) {
        if (exchange_attached && cluster_size_1d(logDY, S, N, K, cus) > 0) return kFused1dCluster;
        if (algo == 7) algo = 0;                                // not applicable here: by size, as for every other value
    }
    if (algo == 8 && (logDY == 7 || logDY == 8)) return kFused1dWide;
    if (algo == 8) algo = 0;
    int pick = algo == 4 ? 2 : algo;
    // lengths 512 / 1024 with 64 channels or more, x and y streamed: the 256-thread matrix-core kernel is 7-16 % ahead of
    // the SIMT kernel on grids of up to four blocks per CU (level or up to 10 % behind on larger ones)
    if (pick == 0)
        pick = (built && items <= cus) ? 2 : ((!long_signal || (K >= 64 && !keep_y && items <= 4L * cus)) ? 3 : 1);
    // small grids, 64 channels or more: eight waves split the K channels of one item (10-16 % ahead of the kernel that
    // shares the spectra through LDS; level at K = 32)
    if (logDY == 8 && (algo == 6 || (algo == 0 && K >= 64 && S * (N / SPLIT_NT) <= cus))) return kFused1dSplit;
    // few blocks: tiles of 32 output channels put twice as many CUs to work (each block still transforms all K inputs)
    if (pick == 2 && (logDY == 7 || logDY == 8) && (algo == 4 || (algo == 0 && S * (N / 32) <= cus))) return kFused1dMfma512Tile32;
    if (pick == 2 && built) return kFused1dMfma512;
    if (pick == 3 && built) return kFused1dMfma256;
    return kFused1dSimt;
}

hipError_t launch_fused_fft_cgemm_ifft(int logDY, long S, int N, int K, const float2* x, const float2* W, float2* y,
                                       float2 alpha, int algo, hipStream_t stream, bool y_is_reread)
{
    // y_is_reread (Y stage of the three-kernel 2D pipeline): the block kernels and the SIMT kernel then leave y in the
    // caches instead of streaming it past them; the other kernels ignore it
    const int keep_y = y_is_reread ? 1 : 0;
    const long cus = cu_count();
    int kernel = pick_fused_1d_kernel(logDY, S, N, K, algo, y_is_reread, cus, exchange_attached(stream));
    if (kernel == kFused1dCluster) {
        const hipError_t e = launch_fused_cluster(S, N, K, cluster_size_1d(logDY, S, N, K, cus), x, W, y, alpha, stream);
        if (e != hipErrorNotReady) return e;
        kernel = pick_fused_1d_kernel(logDY, S, N, K, algo, y_is_reread, cus, false);    // detached in between
    }
    switch (kernel) {
    case kFused1dWave:
        return logDY == 8 ? launch_fused_wave<8>(S, N, K, x, W, y, alpha, stream, keep_y)
                          : launch_fused_wave<7>(S, N, K, x, W, y, alpha, stream, keep_y);
    case kFused1dWide: return launch_fused_wide(logDY, S, N, K, x, W, y, alpha, stream, keep_y);
    case kFused1dSplit: {
        static std::atomic<unsigned long long> served;
        if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(fused_fft_mfma_ifft_split_kernel), SPLIT_LDS, served);
            e != hipSuccess)
            return e;
        if (S * (N / SPLIT_NT) > 0x7fffffffL) return hipErrorInvalidValue;
        hipLaunchKernelGGL(fused_fft_mfma_ifft_split_kernel, dim3((unsigned)(S * (N / SPLIT_NT))), dim3(512), SPLIT_LDS, stream,
                           (int)S, N, K, x, W, y, alpha);
        return hipGetLastError();
    }
    case kFused1dMfma512Tile32:
        return logDY == 8 ? launch_fused_mfma<8, 512, 32>(S, N, K, x, W, y, alpha, stream, keep_y)
                          : launch_fused_mfma<7, 512, 32>(S, N, K, x, W, y, alpha, stream, keep_y);
    case kFused1dMfma512:
        switch (logDY) {
        case 7: return launch_fused_mfma<7, 512>(S, N, K, x, W, y, alpha, stream, keep_y);
        case 8: return launch_fused_mfma<8, 512>(S, N, K, x, W, y, alpha, stream, keep_y);
        case 9: return launch_fused_mfma<9, 512>(S, N, K, x, W, y, alpha, stream, keep_y);
        default: return launch_fused_mfma<10, 512>(S, N, K, x, W, y, alpha, stream, keep_y);
        }
    case kFused1dMfma256:
        switch (logDY) {
        case 7: return launch_fused_mfma<7, 256>(S, N, K, x, W, y, alpha, stream, keep_y);
        case 8: return launch_fused_mfma<8, 256>(S, N, K, x, W, y, alpha, stream, keep_y);
        case 9: return launch_fused_mfma<9, 256>(S, N, K, x, W, y, alpha, stream, keep_y);
        default: return launch_fused_mfma<10, 256>(S, N, K, x, W, y, alpha, stream, keep_y);
        }
    default: return dispatch_fused_1d<true, true>(logDY, S, N, K, x, W, y, alpha, make_float2(0.f, 0.f), stream, keep_y);
    }
}

hipError_t launch_fused_fft_cgemm(int logDY, long S, int N, int K, const float2* x, const float2* W, float2* C,
                                  float2 alpha, float2 beta, hipStream_t stream)
{
    return dispatch_fused_1d<true, false>(logDY, S, N, K, x, W, C, alpha, beta, stream);
}

hipError_t launch_fused_cgemm_ifft(int logDY, long S, int N, int K, const float2* A, const float2* W, float2* y,
                                   float2 alpha, hipStream_t stream)
{
    return dispatch_fused_1d<false, true>(logDY, S, N, K, A, W, y, alpha, make_float2(0.f, 0.f), stream);
}

template <int LOGDY, bool INVERSE>
static hipError_t launch_stride_DY_t(const float2* in, float2* out, long nsig, hipStream_t stream)
{
    using G = Geo1D<LOGDY>;
    const long blocks = (nsig + G::GROUPS - 1) / G::GROUPS;
    if (blocks <= 0 || blocks > 0x7fffffffL) return hipErrorInvalidValue;
    hipLaunchKernelGGL((stride_DY_kernel<LOGDY, INVERSE>), dim3((unsigned)blocks), dim3(256),
                       sizeof(float2) * G::GROUPS * G::EXCH, stream, in, out, nsig);
    return hipGetLastError();
}

hipError_t launch_fft_stride_DY(int logDY, const float2* in, float2* out, long nsig, hipStream_t stream)
{
    switch (logDY) {
    case 7: return launch_stride_DY_t<7, false>(in, out, nsig, stream);
    case 8: return launch_stride_DY_t<8, false>(in, out, nsig, stream);
    case 9: return launch_stride_DY_t<9, false>(in, out, nsig, stream);
    case 10: return launch_stride_DY_t<10, false>(in, out, nsig, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_ifft_stride_DY(int logDY, const float2* in, float2* out, long nsig, hipStream_t stream)
{
    switch (logDY) {
    case 7: return launch_stride_DY_t<7, true>(in, out, nsig, stream);
    case 8: return launch_stride_DY_t<8, true>(in, out, nsig, stream);
    case 9: return launch_stride_DY_t<9, true>(in, out, nsig, stream);
    case 10: return launch_stride_DY_t<10, true>(in, out, nsig, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace tfno
