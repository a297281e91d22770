// Whole-image 2D spectral layer for 256 x 256 grids (the MI355X-first path of the 2D layer).
//
// The reference's "fully fused" 2D variant is three kernels with two HBM round trips of
// half-truncated intermediates (fusion_variants/2D_D_exp_fused_fft_cgemm_ifft/fused_trunc_2D.cu:150-172:
// X transform -> t1[K*bs][64][DY], fused Y stage, t2[N*bs][64][DY] -> X inverse). Here one 1024-thread
// block owns a whole 256 x 256 image, so only fully truncated 64 x 64 spectra (1/16 of the image)
// ever leave the CU:
//
//   fft2d_trunc_256   image (k,b): 256 row FFTs along Y (coalesced 2 KiB rows, 64 modes kept, held in
//                     registers), redistribution through LDS, 64 column FFTs along X (64 modes kept)
//                     -> spec[k][b][4096]                                       reads 512 KiB, writes 32 KiB
//   cgemm_modes       C[n][b][m] = alpha * sum_k W[k][n] spec[k][b][m] on the fp32 matrix cores
//   ifft2d_pad_256    exact mirror -> y[n][b][256][256]                         reads 32 KiB, writes 512 KiB
//
// so x is read once and y written once; padded / discarded modes are never touched in memory.
// The 4096 modes of an image are stored in "lane order": element s*1024 + q*16 + r holds mode
// (p = r + 16 s, q). That order is private to these three kernels (producer and consumer lanes
// coincide, every access is a contiguous 512 B per wavefront) and the GEMM is oblivious to it.
#include "group_fft.h"
#include "kernels.h"

namespace tfno {

namespace {
constexpr int IMG = 256;
constexpr int TPITCH = 66;                       // row pitch (complex) of the 256 x 64 redistribution tile
constexpr int EXCH256 = 16 * 17;                 // exchange region of one 16-lane group
constexpr int LDS2D_ELEMS = 64 * EXCH256 > IMG * TPITCH ? 64 * EXCH256 : IMG * TPITCH;   // exchange regions alias the tile
constexpr size_t LDS2D_BYTES = sizeof(float2) * (size_t)LDS2D_ELEMS;
constexpr size_t LDS2D_FWD_BYTES = sizeof(float2) * (size_t)(LDS2D_ELEMS + kTwLdsSize);

// Row handled by 16-lane group j of wave w in pass `it` (64 groups per block): groups 0/1 of a wave are
// 8 rows apart so the two groups that share an LDS cycle hit disjoint banks in the pitch-66 tile.
__device__ __forceinline__ int row_of(int w, int j, int it)
{
    return 64 * it + ((w & 7) | ((j & 1) << 3) | ((j >> 1) << 4) | ((w >> 3) << 5));
}
// same for a 512-thread block (32 groups, 8 passes)
__device__ __forceinline__ int row_of32(int w, int j, int it)
{
    return 32 * it + (w | ((j & 1) << 3) | ((j >> 1) << 4));
}
}  // namespace

// Forward image kernel. 1024 threads = 64 lane groups = 16 waves per CU (4 per SIMD: the arithmetic
// is issue bound, so full occupancy matters more than registers). A block is persistent over images
// (img = blockIdx.x, += gridDim.x). Each group keeps ONE row in flight: the loads of its next row are
// issued as soon as the first pass has consumed the row registers, so they travel while the exchange
// and the second pass run, across the column pass and across image boundaries. Inter-pass twiddles
// live in LDS to keep the kernel at 128 VGPRs.
__global__ __launch_bounds__(1024) void fft2d_trunc_256_kernel(const float2* __restrict__ x, float2* __restrict__ spec,
                                                               int nimg)
{
    extern __shared__ float2 lds[];
    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, j = lane >> 4, r = lane & 15, g = tid >> 4;
    float2* exch = lds + g * EXCH256;
    float2* twtab = lds + LDS2D_ELEMS;                 // after the exchange regions / tile
    fill_lds_twiddles<8>(twtab, tid, 1024);
    const float2* twrow = twtab + r * kTwLdsPitch;
    __syncthreads();

    const int row0 = row_of(w, j, 0);
    // scalar base + 32-bit lane offset keeps the load addresses out of the vector registers
    const unsigned lane_off = (unsigned)(row0 * IMG + r);
    // x is streamed exactly once: non-temporal loads keep it from evicting the 64x64 spectra, which the
    // next kernel re-reads, out of L2 / Infinity Cache
    auto issue = [&](cpx (&dst)[16], long img, int it) {
        const float2* base = x + (img * IMG + 64 * it) * (long)IMG;
#pragma unroll
        for (int i = 0; i < 16; ++i) dst[i] = load_streaming(&base[lane_off + 16u * i]);
    };

    long img = blockIdx.x;
    cpx v[16];
    if (img < nimg) issue(v, img, 0);
    for (; img < nimg; img += gridDim.x) {
        const long pre = img + gridDim.x < nimg ? img + gridDim.x : img;
        // pass 1: rows (along Y). T[it][s] = mode q = r + 16 s of row row0 + 64 it
        cpx T[4][4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            cpx bb[16], gg[16];
            fft16_stage1<-1>(v, bb);
            // v is dead after the first radix-4 stage: its registers become the landing zone of the next row
            // the last pass already fetches the next image's first row (for the final image: a harmless
            // re-read of its own), so HBM stays busy through the redistribution and the column pass
            if (it + 1 < 4) issue(v, img, it + 1);
            else issue(v, pre, 0);
            fwd_pass1_lds_finish(bb, twrow, gg);
            group_forward_finish<8>(gg, exch, r, T[it]);
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < 4; ++it)
#pragma unroll
            for (int s = 0; s < 4; ++s) lds[(row0 + 64 * it) * TPITCH + r + 16 * s] = T[it][s];
        __syncthreads();
        // pass 2: columns (along X); group g owns column q = g, lane r holds rows r + 16 i
        cpx z[4];
        {
            cpx c[16], gg[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) c[i] = lds[(r + 16 * i) * TPITCH + g];
            __syncthreads();
            fwd_pass1_lds(c, twrow, gg);
            wave_lds_fence();
#pragma unroll
            for (int q = 0; q < 16; ++q) exch[r * 17 + q] = gg[q];
            wave_lds_fence();
            cpx u[16];
#pragma unroll
            for (int tt = 0; tt < 16; ++tt) u[tt] = exch[tt * 17 + r];
            dft16_first4<-1>(u, z);
        }
        // lane order of the retained modes: element s*1024 + q*16 + r  <->  mode (p = r + 16 s, q)
        float2* dst = spec + img * 4096;
#pragma unroll
        for (int s = 0; s < 4; ++s) dst[(unsigned)tid + 1024u * s] = z[s];
    }
}

// Backward image kernel, mirror of the forward one: persistent blocks, 16 waves per CU, twiddles in LDS.
// The 32 KiB spectrum of the next image is fetched (4 registers per lane) while the current image's rows
// are being transformed and stored, so a CU never waits for its input between images.
__global__ __launch_bounds__(1024) void ifft2d_pad_256_kernel(const float2* __restrict__ spec, float2* __restrict__ y,
                                                              int nimg)
{
    extern __shared__ float2 lds[];
    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, j = lane >> 4, r = lane & 15, g = tid >> 4;
    float2* exch = lds + g * EXCH256;
    float2* twtab = lds + LDS2D_ELEMS;
    fill_lds_twiddles<8>(twtab, tid, 1024);
    const float2* twrow = twtab + r * kTwLdsPitch;
    __syncthreads();

    const int row0 = row_of(w, j, 0);
    const unsigned lane_off = (unsigned)(row0 * IMG + r);

    long img = blockIdx.x;
    cpx c[4];
    if (img < nimg) {
        const float2* src = spec + img * 4096;
#pragma unroll
        for (int s = 0; s < 4; ++s) c[s] = src[(unsigned)tid + 1024u * s];
    }
    for (; img < nimg; img += gridDim.x) {
        const long pre = img + gridDim.x < nimg ? img + gridDim.x : img;
        // pass 1: columns (p -> x) of column q = g
        {
            cpx u[16];
            group_backward256_lds(c, twrow, exch, r, u);
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 16; ++i) lds[(r + 16 * i) * TPITCH + g] = u[i];
        }
        // next image's spectrum (for the last image: a harmless re-read of its own)
        {
            const float2* src = spec + pre * 4096;
#pragma unroll
            for (int s = 0; s < 4; ++s) c[s] = src[(unsigned)tid + 1024u * s];
        }
        __syncthreads();
        cpx cc[4][4];
#pragma unroll
        for (int it = 0; it < 4; ++it)
#pragma unroll
            for (int s = 0; s < 4; ++s) cc[it][s] = lds[(row0 + 64 * it) * TPITCH + r + 16 * s];
        __syncthreads();
        // pass 2: rows (q -> y), coalesced 2 KiB row stores.
        // y is written once and not re-read by this layer: non-temporal stores stop half a gigabyte of
        // dirty lines from lingering in the Infinity Cache and being written back under the next kernel's reads
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            cpx yv[16];
            group_backward256_lds(cc[it], twrow, exch, r, yv);
            float2* dst = y + (img * IMG + 64 * it) * (long)IMG;   // uniform base + lane offset + immediates
#pragma unroll
            for (int i = 0; i < 16; ++i) store_streaming(dst + lane_off + 16 * i, yv[i]);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Mode-space complex GEMM on the fp32 matrix cores.
//   C[n][m] = alpha * sum_k W[k + n*K] * A[k][m],   A: [K][Mtot], C: [N][Mtot]  (m contiguous)
// Same contraction as the reference's cgemm / the GEMM phase of its fused kernel
// (fusion_variants/1D_A_exp_fft+cgemm+ifft/cgemm.cuh:4-205, operand layout lda=M, ldb=K, ldc=M),
// expressed as the real product  [Cr;Ci] = [[Wr,-Wi],[Wi,Wr]] [Ar;Ai]  (4-real decomposition) on
// v_mfma_f32_32x32x2_f32: rows = (n, re/im), cols = 32 consecutive m, contraction = (k, re/im).
// One wave owns a 32-m strip and a 64-channel n tile (4 accumulators of 32x32).
// ---------------------------------------------------------------------------------------------
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int GEMM_KC = 64;         // channels per LDS-resident W chunk
constexpr int GEMM_WPITCH = 260;    // floats per k row of the W tile (256 + 4: spreads the k-major fill over banks)
constexpr int GEMM_THREADS = 1024;  // 16 waves: 8 strips of 32 m x 2 halves of the 64-channel n tile
constexpr int GEMM_MBLOCK = 256;    // m per block

// Each wave owns a 32-m strip and one half (32 channels) of the n tile, i.e. two 32x32 accumulators. The four
// waves that share a SIMD get descending issue priorities, so their matrix-core phases finish staggered and
// the stores of one wave drain while the next wave still computes (otherwise all stores hit HBM at the end).
__global__ __launch_bounds__(GEMM_THREADS) void cgemm_modes_kernel(const float2* __restrict__ A,
                                                                   const float2* __restrict__ W, float2* __restrict__ C,
                                                                   long Mtot, int N, int K, float2 alpha)
{
    // sW[k*260 + n'*2 + c] = Wreal[n' = 2 n + c'][k' = 2 k + c]:  {Wr, -Wi} for c'=0, {Wi, Wr} for c'=1
    __shared__ float sW[GEMM_KC * GEMM_WPITCH];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, col = lane & 31, half = lane >> 5;
    const int strip = wave >> 1, nh = wave & 1;
    const int n0 = blockIdx.y * 64;
    switch (wave >> 2) {                      // waves w, w+4, w+8, w+12 share a SIMD
    case 0: __builtin_amdgcn_s_setprio(3); break;
    case 1: __builtin_amdgcn_s_setprio(2); break;
    case 2: __builtin_amdgcn_s_setprio(1); break;
    default: __builtin_amdgcn_s_setprio(0); break;
    }

    floatx16 acc[2];
#pragma unroll
    for (int tI = 0; tI < 2; ++tI)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[tI][e] = 0.f;

    for (int kc = 0; kc < K; kc += GEMM_KC) {
        const int kn = (K - kc) < GEMM_KC ? (K - kc) : GEMM_KC;
        // lane (col, half) feeds A[kc + kk + half][m0 + col] as {re, im}; all loads of the chunk are issued
        // before the W tile is built so their latency hides behind it
        // (scalar base per k pair + one 32-bit lane offset keeps the 32 addresses out of the vector registers)
        const unsigned lane_off = (unsigned)(half * Mtot) + (unsigned)(strip * 32 + col);
        float2 bv[GEMM_KC / 2];
#pragma unroll
        for (int q = 0; q < GEMM_KC / 2; ++q) {
            const float2* base = A + (long)(kc + 2 * q) * Mtot + (long)blockIdx.x * GEMM_MBLOCK;
            bv[q] = (2 * q < kn) ? base[lane_off] : make_float2(0.f, 0.f);
        }
        __syncthreads();
        // all W loads of the tile are issued before the first LDS store (one round trip)
        constexpr int WPT = GEMM_KC * 64 / GEMM_THREADS;
        float2 wv[WPT];
#pragma unroll
        for (int u = 0; u < WPT; ++u) {
            const int idx = tid + u * GEMM_THREADS;
            const int k = idx % GEMM_KC, n = idx / GEMM_KC;   // k fastest: coalesced reads of W[k + n*K]
            wv[u] = (k < kn) ? W[(kc + k) + (long)(n0 + n) * K] : make_float2(0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < WPT; ++u) {
            const int idx = tid + u * GEMM_THREADS;
            const int k = idx % GEMM_KC, n = idx / GEMM_KC;
            const float2 w = make_float2(wv[u].x * alpha.x - wv[u].y * alpha.y, wv[u].x * alpha.y + wv[u].y * alpha.x);
            *reinterpret_cast<float4*>(&sW[k * GEMM_WPITCH + 4 * n]) = make_float4(w.x, -w.y, w.y, w.x);
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < GEMM_KC / 2; ++q) {
#pragma unroll
            for (int tI = 0; tI < 2; ++tI) {
                float2 a = *reinterpret_cast<const float2*>(
                    &sW[(2 * q + half) * GEMM_WPITCH + ((nh * 2 + tI) * 32 + col) * 2]);
                acc[tI] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, bv[q].x, acc[tI], 0, 0, 0);
                acc[tI] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, bv[q].y, acc[tI], 0, 0, 0);
            }
            // keep the W-operand reads next to their matrix instructions (hoisting all 64 of them spills)
            if ((q & 1) == 1) __builtin_amdgcn_sched_barrier(0);
        }
    }
    // D[row = 8 i + 4 half + jj*2 + c'][col]: row = 2 n_local + c'
#pragma unroll
    for (int tI = 0; tI < 2; ++tI)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                float2* base = C + (long)(n0 + (nh * 2 + tI) * 16 + 4 * i + jj) * Mtot + (long)blockIdx.x * GEMM_MBLOCK;
                base[(unsigned)(2 * half * Mtot) + (unsigned)(strip * 32 + col)] =
                    make_float2(acc[tI][4 * i + 2 * jj], acc[tI][4 * i + 2 * jj + 1]);
            }
}

static int cu_count()
{
    static int cus = 0;
    if (!cus) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
        else cus = 256;
    }
    return cus;
}

hipError_t launch_fft2d_trunc_256(const float2* x, float2* spec, long nimg, hipStream_t stream)
{
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fft2d_trunc_256_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS2D_FWD_BYTES);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    // one persistent block per CU (the LDS tile allows exactly one resident block per CU)
    const long blocks = nimg < cu_count() ? nimg : cu_count();
    hipLaunchKernelGGL(fft2d_trunc_256_kernel, dim3((unsigned)blocks), dim3(1024), LDS2D_FWD_BYTES, stream, x, spec,
                       (int)nimg);
    return hipGetLastError();
}

hipError_t launch_ifft2d_pad_256(const float2* spec, float2* y, long nimg, hipStream_t stream)
{
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(ifft2d_pad_256_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS2D_FWD_BYTES);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const long blocks = nimg < cu_count() ? nimg : cu_count();
    hipLaunchKernelGGL(ifft2d_pad_256_kernel, dim3((unsigned)blocks), dim3(1024), LDS2D_FWD_BYTES, stream, spec, y,
                       (int)nimg);
    return hipGetLastError();
}

hipError_t launch_cgemm_modes(const float2* A, const float2* W, float2* C, long Mtot, int N, int K, float2 alpha,
                              hipStream_t stream)
{
    if (Mtot % GEMM_MBLOCK != 0 || Mtot >= (1L << 27) || N % 64 != 0 || K % 2 != 0) return hipErrorInvalidValue;
    dim3 grid((unsigned)(Mtot / GEMM_MBLOCK), (unsigned)(N / 64), 1);
    hipLaunchKernelGGL(cgemm_modes_kernel, grid, dim3(GEMM_THREADS), 0, stream, A, W, C, Mtot, N, K, alpha);
    return hipGetLastError();
}

}  // namespace tfno
