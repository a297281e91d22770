// Fused 1D spectral layer: forward FFT along DY -> keep 64 modes -> complex GEMM over the channel
// dimension -> zero-pad -> backward FFT, in ONE kernel with no HBM round trip in between.
//
// Replaces fused_fft_cgemm_ifft_{7,8} of the reference
// (fusion_variants/1D_D_exp_fused_fft_cgemm_ifft/fused_fft_cgemm_ifft_7.cuh:9-222): same operands
//   x[K][S][DY]  (signal (k,s) at (k*S+s)*DY),  W[k + n*K],  y[N][S][DY],  M = 64*S,
// same grid (S, N/64), block 256, and the same "block traverses K" schedule, re-derived for wave64:
//   * an L = DY/16 lane group owns one signal; a 256-thread block transforms 256/L channels at once
//     (the reference does 8), so the K loop advances in chunks of 16 (DY=256) or 32 (DY=128) channels;
//   * the thread that accumulates C[m][n] is the thread that later needs it for the backward
//     transform, so the GEMM result never passes through LDS (the reference stages it in 8 rounds,
//     fused_fft_cgemm_ifft_7.cuh:203-218);
//   * exchange buffers are padded (row pitch 17 complex) for the 64-bank LDS of CDNA4.
#include "group_fft.h"
#include "kernels.h"

namespace tfno {

template <int LOGDY>
__global__ __launch_bounds__(256) void fused_fft_cgemm_ifft_kernel(int S, int N, int K, const float2* __restrict__ x,
                                                                   const float2* __restrict__ W, float2* __restrict__ y,
                                                                   float2 alpha)
{
    using G = Geo1D<LOGDY>;
    constexpr int DY = G::DY, L = G::L, GROUPS = G::GROUPS, MM = G::MM, NN = G::NN;
    extern __shared__ float2 lds[];
    float2* sA = lds;                                  // [GROUPS][64]   truncated spectra of the K chunk
    float2* sW = sA + GROUPS * G::SA_PITCH;            // [GROUPS][64]   W chunk, sW[kk][n]
    float2* exch_all = sW + GROUPS * 64;

    const int tid = threadIdx.x;
    const int g = tid / L, t = tid % L;
    const long s = blockIdx.x;
    const int n0 = blockIdx.y * 64;
    float2* exch = exch_all + g * G::EXCH;

    cpx tw[16];
    load_lane_twiddles<LOGDY>(t, tw);

    cpx acc[MM][NN];
#pragma unroll
    for (int a = 0; a < MM; ++a)
#pragma unroll
        for (int b = 0; b < NN; ++b) acc[a][b] = make_float2(0.f, 0.f);

    for (int kc = 0; kc < K; kc += GROUPS) {
        const int k = kc + g;
        cpx out[MM];
        if (k < K) {
            const float2* src = x + ((long)k * S + s) * DY + t;
            cpx v[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) v[i] = src[L * i];
            group_forward<LOGDY>(v, tw, exch, t, out);
        } else {
#pragma unroll
            for (int a = 0; a < MM; ++a) out[a] = make_float2(0.f, 0.f);
        }
#pragma unroll
        for (int a = 0; a < MM; ++a) sA[g * G::SA_PITCH + t + L * a] = out[a];
        // W chunk: GROUPS x 64 elements, consecutive threads read consecutive k (contiguous in memory)
#pragma unroll
        for (int j = 0; j < (GROUPS * 64) / 256; ++j) {
            int idx = tid + 256 * j;
            int kk = idx % GROUPS, n = idx / GROUPS;
            float2 w = make_float2(0.f, 0.f);
            if (kc + kk < K) w = W[(kc + kk) + (long)(n0 + n) * K];
            sW[kk * 64 + n] = w;
        }
        __syncthreads();
#pragma unroll 4
        for (int kk = 0; kk < GROUPS; ++kk) {
            cpx a[MM], b[NN];
#pragma unroll
            for (int i = 0; i < MM; ++i) a[i] = sA[kk * G::SA_PITCH + t + L * i];
#pragma unroll
            for (int j = 0; j < NN; ++j) b[j] = sW[kk * 64 + g + GROUPS * j];
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
        cpx c[MM], yv[16];
#pragma unroll
        for (int i = 0; i < MM; ++i) c[i] = cmul(acc[i][j], alpha);
        group_backward<LOGDY>(c, tw, exch, t, yv);
        float2* dst = y + ((long)n * S + s) * DY + t;
#pragma unroll
        for (int i = 0; i < 16; ++i) dst[L * i] = yv[i];
    }
}

template <int LOGDY>
static hipError_t launch_fused_1d(long S, int N, int K, const float2* x, const float2* W, float2* y, float2 alpha,
                                  hipStream_t stream)
{
    using G = Geo1D<LOGDY>;
    dim3 grid((unsigned)S, (unsigned)(N / 64), 1), block(256, 1, 1);
    hipLaunchKernelGGL(fused_fft_cgemm_ifft_kernel<LOGDY>, grid, block, G::LDS_BYTES, stream, (int)S, N, K, x, W, y,
                       alpha);
    return hipGetLastError();
}

hipError_t launch_fused_fft_cgemm_ifft(int logDY, long S, int N, int K, const float2* x, const float2* W, float2* y,
                                       float2 alpha, hipStream_t stream)
{
    switch (logDY) {
    case 7: return launch_fused_1d<7>(S, N, K, x, W, y, alpha, stream);
    case 8: return launch_fused_1d<8>(S, N, K, x, W, y, alpha, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace tfno
