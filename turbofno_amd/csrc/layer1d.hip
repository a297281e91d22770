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

// FUSE_FWD: the A operand is produced by forward transforms of x (variants B and D); otherwise it is read from
//           the column-major matrix A[m + k*M] (variant C).
// FUSE_INV: the product goes straight into zero-padded backward transforms (variants C and D); otherwise it is
//           stored as C[m + n*M] = alpha*A*W + beta*C (variant B).
template <int LOGDY, bool FUSE_FWD, bool FUSE_INV>
__global__ __launch_bounds__(256) void fused_fft_cgemm_ifft_kernel(int S, int N, int K, const float2* __restrict__ x,
                                                                   const float2* __restrict__ W, float2* __restrict__ y,
                                                                   float2 alpha, float2 beta)
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
    const long M = 64L * S;
    float2* exch = exch_all + g * G::EXCH;

    cpx tw[16];
    load_lane_twiddles<LOGDY>(t, tw);

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
        if constexpr (FUSE_INV) {
            cpx c[MM], yv[16];
#pragma unroll
            for (int i = 0; i < MM; ++i) c[i] = cmul(acc[i][j], alpha);
            group_backward<LOGDY>(c, tw, exch, t, yv);
            float2* dst = y + ((long)n * S + s) * DY + t;
#pragma unroll
            for (int i = 0; i < 16; ++i) dst[L * i] = yv[i];
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
    float2* exch = lds + g * G::EXCH;
    cpx tw[16];
    load_lane_twiddles<LOGDY>(t, tw);
    if (sig >= nsig) return;
    if constexpr (!INVERSE) {
        const float2* src = in + sig * DY + t;
        cpx v[16], o[MM];
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = src[L * i];
        group_forward<LOGDY>(v, tw, exch, t, o);
        float2* dst = out + sig * 64 + t;
#pragma unroll
        for (int a = 0; a < MM; ++a) dst[L * a] = o[a];
    } else {
        const float2* src = in + sig * 64 + t;
        cpx c[MM], yv[16];
#pragma unroll
        for (int a = 0; a < MM; ++a) c[a] = src[L * a];
        group_backward<LOGDY>(c, tw, exch, t, yv);
        float2* dst = out + sig * DY + t;
#pragma unroll
        for (int i = 0; i < 16; ++i) dst[L * i] = yv[i];
    }
}

template <int LOGDY, bool FUSE_FWD, bool FUSE_INV>
static hipError_t launch_fused_1d(long S, int N, int K, const float2* x, const float2* W, float2* y, float2 alpha,
                                  float2 beta, hipStream_t stream)
{
    using G = Geo1D<LOGDY>;
    dim3 grid((unsigned)S, (unsigned)(N / 64), 1), block(256, 1, 1);
    hipLaunchKernelGGL((fused_fft_cgemm_ifft_kernel<LOGDY, FUSE_FWD, FUSE_INV>), grid, block, G::LDS_BYTES, stream, (int)S,
                       N, K, x, W, y, alpha, beta);
    return hipGetLastError();
}

template <bool FUSE_FWD, bool FUSE_INV>
static hipError_t dispatch_fused_1d(int logDY, long S, int N, int K, const float2* x, const float2* W, float2* y,
                                    float2 alpha, float2 beta, hipStream_t stream)
{
    switch (logDY) {
    case 7: return launch_fused_1d<7, FUSE_FWD, FUSE_INV>(S, N, K, x, W, y, alpha, beta, stream);
    case 8: return launch_fused_1d<8, FUSE_FWD, FUSE_INV>(S, N, K, x, W, y, alpha, beta, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_fused_fft_cgemm_ifft(int logDY, long S, int N, int K, const float2* x, const float2* W, float2* y,
                                       float2 alpha, hipStream_t stream)
{
    return dispatch_fused_1d<true, true>(logDY, S, N, K, x, W, y, alpha, make_float2(0.f, 0.f), stream);
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
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_ifft_stride_DY(int logDY, const float2* in, float2* out, long nsig, hipStream_t stream)
{
    switch (logDY) {
    case 7: return launch_stride_DY_t<7, true>(in, out, nsig, stream);
    case 8: return launch_stride_DY_t<8, true>(in, out, nsig, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace tfno
