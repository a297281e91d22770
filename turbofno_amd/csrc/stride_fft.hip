// X-axis transforms of the three-kernel 2D pipeline: forward FFT along DX (element stride DY) with
// truncation to the first 64 rows, and its mirror, zero-padding 64 rows to DX and transforming back.
//
// Replace fft_N_stride / ifft_N_stride of the reference's missing TurboFFT submodule, launched at
// fusion_variants/2D_D_exp_fused_fft_cgemm_ifft/fused_trunc_2D.cu:153-160 and :170:
//   forward   in[sig][DX][DY]  -> out[sig][64][DY]
//   backward  in[sig][64][DY]  -> out[sig][DX][DY]
// A block owns COLS = 16 or 32 adjacent columns (128 or 256 contiguous bytes per row, whole cache lines; the
// reference uses 4 columns = 32 bytes) and all DX rows; thread (yl, t) holds rows t + L*i of column yl in
// registers, runs the 16-point pass there, and the single exchange goes through LDS laid out
// [t][r][yl] so that both the writes and the reads are conflict free on 64 banks.
#include "fft_codelets.h"
#include "kernels.h"

namespace tfno {

template <int LOGDX, int COLS_> struct GeoStride {
    static constexpr int DX = 1 << LOGDX;
    static constexpr int L = DX / 16;
    static constexpr int COLS = COLS_;                 // adjacent columns per block: 8 * COLS contiguous bytes per row
    static constexpr int THREADS = COLS * L;
    static constexpr size_t LDS_BYTES = sizeof(float2) * (size_t)(L * 17 * COLS);
};

template <int LOGDX, int COLS>
__global__ __launch_bounds__((GeoStride<LOGDX, COLS>::THREADS)) void fft_stride_kernel(const float2* __restrict__ in,
                                                                                    float2* __restrict__ out, int DY)
{
    using G = GeoStride<LOGDX, COLS>;
    constexpr int DX = G::DX, L = G::L;
    extern __shared__ float2 lds[];
    const int tid = threadIdx.x, yl = tid % COLS, t = tid / COLS;
    const long col = (long)blockIdx.x * COLS + yl;
    const long sig = col / DY;
    const int y = (int)(col % DY);

    cpx tw[16], v[16], g[16];
    load_lane_twiddles<LOGDX>(t, tw);
    const float2* src = in + (sig * DX + t) * DY + y;
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = src[(long)L * i * DY];
    fwd_pass1(v, tw, g);
#pragma unroll
    for (int r = 0; r < 16; ++r) lds[(t * 17 + r) * COLS + yl] = g[r];
    __syncthreads();
    float2* dst = out + sig * 64 * DY + y;
    if constexpr (L >= 32) {
        // lengths 512 / 1024: pruned second pass with a second, small exchange (wide_forward_inner / _outer on this
        // kernel's [t][r][yl] layout); thread (yl, t) ends up with rows wide_mode<L>(t, mm)
        cpx inner[4], o[64 / L];
        wide_forward_inner<L>(lds + yl, COLS, t, inner);
        __syncthreads();
#pragma unroll
        for (int c = 0; c < 4; ++c) lds[wide_swap_index<L>(t / (L / 16), c, t % (L / 16)) * COLS + yl] = inner[c];
        __syncthreads();
        wide_forward_outer<L>(lds + yl, COLS, t, o);
#pragma unroll
        for (int mm = 0; mm < 64 / L; ++mm) dst[(long)wide_mode<L>(t, mm) * DY] = o[mm];
    } else if constexpr (L == 16) {
        cpx u[16], o[4];
#pragma unroll
        for (int tt = 0; tt < 16; ++tt) u[tt] = lds[(tt * 17 + t) * COLS + yl];
        dft16_first4<-1>(u, o);
#pragma unroll
        for (int s = 0; s < 4; ++s) dst[(long)(t + 16 * s) * DY] = o[s];
    } else {
        cpx u0[8], u1[8], o0[4], o1[4];
#pragma unroll
        for (int tt = 0; tt < 8; ++tt) {
            u0[tt] = lds[(tt * 17 + t) * COLS + yl];
            u1[tt] = lds[(tt * 17 + t + 8) * COLS + yl];
        }
        dft8_first4<-1>(u0, o0);
        dft8_first4<-1>(u1, o1);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            dst[(long)(t + 16 * s) * DY] = o0[s];
            dst[(long)(t + 8 + 16 * s) * DY] = o1[s];
        }
    }
}

// Forward kernel of lengths 512 / 1024, persistent: a block walks panels blockIdx.x, + gridDim.x, ... and issues the loads
// of its next panel as soon as the first pass has consumed the registers of the current one. At these lengths only one or
// two blocks fit a CU (the exchange array), so without the look-ahead the memory system idles while a block computes.
template <int LOGDX, int COLS>
__global__ __launch_bounds__((GeoStride<LOGDX, COLS>::THREADS)) void fft_stride_persistent_kernel(const float2* __restrict__ in,
                                                                                               float2* __restrict__ out, int DY,
                                                                                               long npanels)
{
    using G = GeoStride<LOGDX, COLS>;
    constexpr int DX = G::DX, L = G::L;
    static_assert(LOGDX >= 9, "lengths up to 256 use fft_stride_kernel");
    extern __shared__ float2 lds[];
    const int tid = threadIdx.x, yl = tid % COLS, t = tid / COLS;
    cpx tw[16], v[16];
    load_lane_twiddles<LOGDX>(t, tw);
    auto fetch = [&](long panel) {
        const long col = panel * COLS + yl;
        const float2* src = in + ((col / DY) * DX + t) * DY + (int)(col % DY);
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = src[(long)L * i * DY];
    };
    long panel = blockIdx.x;
    if (panel < npanels) fetch(panel);
    for (; panel < npanels; panel += gridDim.x) {
        const long col = panel * COLS + yl;
        float2* dst = out + (col / DY) * 64 * DY + (int)(col % DY);
        cpx g[16];
        fwd_pass1(v, tw, g);
        if (panel + gridDim.x < npanels) fetch(panel + gridDim.x);
#pragma unroll
        for (int r = 0; r < 16; ++r) lds[(t * 17 + r) * COLS + yl] = g[r];
        __syncthreads();
        cpx inner[4], o[64 / L];
        wide_forward_inner<L>(lds + yl, COLS, t, inner);
        __syncthreads();
#pragma unroll
        for (int c = 0; c < 4; ++c) lds[wide_swap_index<L>(t / (L / 16), c, t % (L / 16)) * COLS + yl] = inner[c];
        __syncthreads();
        wide_forward_outer<L>(lds + yl, COLS, t, o);
#pragma unroll
        for (int mm = 0; mm < 64 / L; ++mm) dst[(long)wide_mode<L>(t, mm) * DY] = o[mm];
        __syncthreads();                                     // the exchange array is free for the next panel
    }
}

template <int LOGDX, int COLS>
__global__ __launch_bounds__((GeoStride<LOGDX, COLS>::THREADS)) void ifft_stride_kernel(const float2* __restrict__ in,
                                                                                     float2* __restrict__ out, int DY)
{
    using G = GeoStride<LOGDX, COLS>;
    constexpr int DX = G::DX, L = G::L;
    extern __shared__ float2 lds[];
    const int tid = threadIdx.x, yl = tid % COLS, t = tid / COLS;
    const long col = (long)blockIdx.x * COLS + yl;
    const long sig = col / DY;
    const int y = (int)(col % DY);

    cpx tw[16];
    load_lane_twiddles<LOGDX>(t, tw);
    const float2* src = in + sig * 64 * DY + y;
    if constexpr (L >= 32) {
#pragma unroll
        for (int mm = 0; mm < 64 / L; ++mm) lds[(t + L * mm) * COLS + yl] = src[(long)(t + L * mm) * DY];
    } else if constexpr (L == 16) {
        cpx c[4], h[16];
#pragma unroll
        for (int s = 0; s < 4; ++s) c[s] = src[(long)(t + 16 * s) * DY];
        dft16_pad4<+1>(c, h);
#pragma unroll
        for (int tt = 0; tt < 16; ++tt) lds[(tt * 17 + t) * COLS + yl] = h[tt];
    } else {
        cpx c0[4], c1[4], h0[8], h1[8];
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            c0[s] = src[(long)(t + 16 * s) * DY];
            c1[s] = src[(long)(t + 8 + 16 * s) * DY];
        }
        dft8_pad4<+1>(c0, h0);
        dft8_pad4<+1>(c1, h1);
#pragma unroll
        for (int tt = 0; tt < 8; ++tt) {
            lds[(tt * 17 + t) * COLS + yl] = h0[tt];
            lds[(tt * 17 + t + 8) * COLS + yl] = h1[tt];
        }
    }
    __syncthreads();
    cpx e[16], yv[16];
    if constexpr (L >= 32) {
        // first-pass inputs from the 64 retained rows: twiddle once per four row groups, 4-point transform, second small
        // exchange (wide_backward_partial / wide_back_index on this kernel's [.][yl] layout)
        cpx part[16];
        wide_backward_partial<L>(lds + yl, COLS, t, part);
        __syncthreads();                                 // every thread has read the 64 rows
#pragma unroll
        for (int k = 0; k < 16; ++k) lds[wide_back_index<L>(t, k) * COLS + yl] = part[k];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 16; ++r) e[r] = lds[(t * 17 + r) * COLS + yl];
    } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) e[r] = lds[(t * 17 + r) * COLS + yl];
    }
    inv_pass2(e, tw, yv);
    float2* dst = out + (sig * DX + t) * DY + y;
#pragma unroll
    for (int i = 0; i < 16; ++i) store_streaming(dst + (long)L * i * DY, yv[i]);
}

// Backward kernel of lengths 512 / 1024, persistent: a block walks panels blockIdx.x, + gridDim.x, ... and fetches the retained rows of
// its next panel (2 to 8 values per thread) as soon as those of the current one are in LDS. Inside the three-kernel
// pipeline these rows come from HBM while the memory system is saturated with this kernel's own stores; without the
// look-ahead every block began with that exposed latency (length 512, 1024 images: 587 us in the pipeline against 416 us
// with the input resident in the Infinity Cache).
template <int LOGDX, int COLS>
__global__ __launch_bounds__((GeoStride<LOGDX, COLS>::THREADS)) void ifft_stride_persistent_kernel(const float2* __restrict__ in,
                                                                                     float2* __restrict__ out, int DY, long npanels,
                                                                                     int even_share)
{
    using G = GeoStride<LOGDX, COLS>;
    constexpr int DX = G::DX, L = G::L;
    static_assert(LOGDX >= 9, "lengths up to 256 use ifft_stride_kernel");
    constexpr int NIN = 64 / L < 4 ? (L == 8 ? 8 : 4) : 64 / L;   // retained rows per thread: 2 / 1 (L = 32 / 64), 4 (16), 8 (8)
    extern __shared__ float2 lds[];
    const int tid = threadIdx.x, yl = tid % COLS, t = tid / COLS;

    cpx tw[16];
    load_lane_twiddles<LOGDX>(t, tw);
    // rows of the retained block a thread reads, in the order its first step wants them
    auto fetch = [&](cpx (&c)[NIN], long panel) {
        const long col = panel * COLS + yl;
        const float2* src = in + (col / DY) * 64 * DY + (int)(col % DY);
        if constexpr (L >= 32) {
#pragma unroll
            for (int mm = 0; mm < 64 / L; ++mm) c[mm] = src[(long)(t + L * mm) * DY];
        } else if constexpr (L == 16) {
#pragma unroll
            for (int s = 0; s < 4; ++s) c[s] = src[(long)(t + 16 * s) * DY];
        } else {
#pragma unroll
            for (int s = 0; s < 4; ++s) { c[s] = src[(long)(t + 16 * s) * DY]; c[4 + s] = src[(long)(t + 8 + 16 * s) * DY]; }
        }
    };
    cpx c[NIN];
    // The odd XCDs of an MI355X store about a fifth slower than the even ones, and workgroup b runs on XCD b mod 8: the
    // blocks 2p and 2p + 1 share the panels p, p + pairs, p + 2 pairs, ... of their pair even_share : 32 - even_share
    // (17 : 15 there, 16 : 16 on other parts; the even block takes the first ones), so that both end together. An odd
    // grid keeps the even split.
    long panel = blockIdx.x, step = gridDim.x, last = npanels;
    if ((gridDim.x & 1) == 0) {
        const long pairs = gridDim.x >> 1, pr = blockIdx.x >> 1;
        const long J = (npanels - pr + pairs - 1) / pairs;          // panels of this pair (pr < npanels: the grid is no larger)
        const long even = (J * even_share + kEvenShareDen / 2) / kEvenShareDen;
        step = pairs;
        panel = (blockIdx.x & 1) ? pr + pairs * even : pr;
        last = (blockIdx.x & 1) ? npanels : pr + pairs * even;
        if (last > npanels) last = npanels;
    }
    const long npanels_mine = last;
    if (panel < npanels_mine) fetch(c, panel);
    for (; panel < npanels_mine; panel += step) {
        const long col = panel * COLS + yl;
        const long sig = col / DY;
        const int y = (int)(col % DY);
        if constexpr (L >= 32) {
#pragma unroll
            for (int mm = 0; mm < 64 / L; ++mm) lds[(t + L * mm) * COLS + yl] = c[mm];
        } else if constexpr (L == 16) {
            cpx c4[4], h[16];
#pragma unroll
            for (int s = 0; s < 4; ++s) c4[s] = c[s];
            dft16_pad4<+1>(c4, h);
#pragma unroll
            for (int tt = 0; tt < 16; ++tt) lds[(tt * 17 + t) * COLS + yl] = h[tt];
        } else {
            cpx c0[4], c1[4], h0[8], h1[8];
#pragma unroll
            for (int s = 0; s < 4; ++s) { c0[s] = c[s]; c1[s] = c[4 + s]; }
            dft8_pad4<+1>(c0, h0);
            dft8_pad4<+1>(c1, h1);
#pragma unroll
            for (int tt = 0; tt < 8; ++tt) {
                lds[(tt * 17 + t) * COLS + yl] = h0[tt];
                lds[(tt * 17 + t + 8) * COLS + yl] = h1[tt];
            }
        }
        if (panel + step < npanels_mine) fetch(c, panel + step);           // look-ahead: travels under the rest of this panel
        __syncthreads();
        cpx e[16], yv[16];
        if constexpr (L >= 32) {
            // first-pass inputs from the 64 retained rows: twiddle once per four row groups, 4-point transform, second small
            // exchange (wide_backward_partial / wide_back_index on this kernel's [.][yl] layout)
            cpx part[16];
            wide_backward_partial<L>(lds + yl, COLS, t, part);
            __syncthreads();                                 // every thread has read the 64 rows
#pragma unroll
            for (int k = 0; k < 16; ++k) lds[wide_back_index<L>(t, k) * COLS + yl] = part[k];
            __syncthreads();
#pragma unroll
            for (int r = 0; r < 16; ++r) e[r] = lds[(t * 17 + r) * COLS + yl];
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) e[r] = lds[(t * 17 + r) * COLS + yl];
        }
        inv_pass2(e, tw, yv);
        float2* dst = out + (sig * DX + t) * DY + y;
#pragma unroll
        for (int i = 0; i < 16; ++i) store_streaming(dst + (long)L * i * DY, yv[i]);
        __syncthreads();                                     // the exchange array is free for the next panel
    }
}

template <int LOGDX, bool INVERSE, int COLS>
static hipError_t launch_stride_c(const float2* in, float2* out, int DY, long nsig, hipStream_t stream)
{
    using G = GeoStride<LOGDX, COLS>;
    long blocks = nsig * DY / COLS;
    if (blocks <= 0 || blocks > 0x7fffffffL || DY % COLS != 0) return hipErrorInvalidValue;
    dim3 grid((unsigned)blocks, 1, 1), block(G::THREADS, 1, 1);
    if constexpr (G::LDS_BYTES > 64 * 1024) {
        static std::atomic<unsigned long long> served;
        const void* fn;                                  // the kernel that is launched below
        if constexpr (INVERSE ? LOGDX >= 9 : LOGDX >= 10)
            fn = INVERSE ? reinterpret_cast<const void*>(ifft_stride_persistent_kernel<LOGDX, COLS>)
                         : reinterpret_cast<const void*>(fft_stride_persistent_kernel<LOGDX, COLS>);
        else
            fn = INVERSE ? reinterpret_cast<const void*>(ifft_stride_kernel<LOGDX, COLS>)
                         : reinterpret_cast<const void*>(fft_stride_kernel<LOGDX, COLS>);
        if (hipError_t e = allow_dynamic_lds(fn, G::LDS_BYTES, served); e != hipSuccess) return e;
    }
    constexpr bool PERSISTENT = INVERSE ? LOGDX >= 9 : LOGDX >= 10;   // forward, length 512: no gain measured
    if constexpr (PERSISTENT) {
        // persistent grid: as many blocks as are resident at once. Lengths up to 256 keep one block per panel: their
        // input (at most 128 MiB at bs = 16) is still in the caches when the kernel runs, and the persistent form was
        // measured 3-8 % slower there.
        static std::atomic<int> per_cu[64];
        int dev = 0;
        if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
        int occ = per_cu[dev & 63].load(std::memory_order_relaxed);
        if (occ <= 0) {
            const hipError_t e = INVERSE ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, ifft_stride_persistent_kernel<LOGDX, COLS>,
                                                                                        G::THREADS, G::LDS_BYTES)
                                         : hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, fft_stride_persistent_kernel<LOGDX, COLS>,
                                                                                        G::THREADS, G::LDS_BYTES);
            if (e != hipSuccess) return e;
            if (occ <= 0) occ = 1;
            per_cu[dev & 63].store(occ, std::memory_order_relaxed);
        }
        const long resident = (long)occ * cu_count();
        const dim3 pgrid((unsigned)(blocks < resident ? blocks : resident));
        if (INVERSE) hipLaunchKernelGGL((ifft_stride_persistent_kernel<LOGDX, COLS>), pgrid, block, G::LDS_BYTES, stream, in, out, DY, blocks, even_share_parts());
        else hipLaunchKernelGGL((fft_stride_persistent_kernel<LOGDX, COLS>), pgrid, block, G::LDS_BYTES, stream, in, out, DY, blocks);
        return hipGetLastError();
    }
    if (INVERSE) hipLaunchKernelGGL((ifft_stride_kernel<LOGDX, COLS>), grid, block, G::LDS_BYTES, stream, in, out, DY);
    else hipLaunchKernelGGL((fft_stride_kernel<LOGDX, COLS>), grid, block, G::LDS_BYTES, stream, in, out, DY);
    return hipGetLastError();
}

// Columns per block: 16 (one 128-byte line per row) in general; the backward kernels of lengths up to 256 take 32
// (256 contiguous bytes per row, 10 % faster: 153 -> 136 us for 1024 images of 256 x 256), where the doubled exchange
// buffer still leaves two blocks per CU. Wider panels did not help the forward kernels.
template <int LOGDX, bool INVERSE>
static hipError_t launch_stride_t(const float2* in, float2* out, int DY, long nsig, hipStream_t stream)
{
    if constexpr (INVERSE && LOGDX <= 8) {
        if (DY % 32 == 0) return launch_stride_c<LOGDX, INVERSE, 32>(in, out, DY, nsig, stream);
    }
    return launch_stride_c<LOGDX, INVERSE, 16>(in, out, DY, nsig, stream);
}

hipError_t launch_fft_stride(int logDX, const float2* in, float2* out, int DY, long nsig, hipStream_t stream)
{
    switch (logDX) {
    case 7: return launch_stride_t<7, false>(in, out, DY, nsig, stream);
    case 8: return launch_stride_t<8, false>(in, out, DY, nsig, stream);
    case 9: return launch_stride_t<9, false>(in, out, DY, nsig, stream);
    case 10: return launch_stride_t<10, false>(in, out, DY, nsig, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_ifft_stride(int logDX, const float2* in, float2* out, int DY, long nsig, hipStream_t stream)
{
    switch (logDX) {
    case 7: return launch_stride_t<7, true>(in, out, DY, nsig, stream);
    case 8: return launch_stride_t<8, true>(in, out, DY, nsig, stream);
    case 9: return launch_stride_t<9, true>(in, out, DY, nsig, stream);
    case 10: return launch_stride_t<10, true>(in, out, DY, nsig, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace tfno
