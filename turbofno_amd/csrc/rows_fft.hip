// Y-axis transforms of the rows-first 2D pipeline: the contiguous axis is transformed first (forward) and last
// (backward), so that the two kernels that touch the full-size arrays x and y move whole rows of 8 * DY contiguous
// bytes, and the X axis is left to the fused 1D kernel on the truncated intermediates:
//   forward   in[img][DX][DY]  -> out[img][64][DX]     rows transformed along DY, 64 modes kept, stored transposed
//   backward  in[img][64][DX]  -> out[img][DX][DY]     read transposed, 64 modes zero-padded to DY, transformed back
// The transposed intermediates out[img][ky][x] are exactly the layout x[k][S][DX], S = bs * 64, of the fused 1D layer
// (fused_fft_cgemm_ifft_* of the reference, launched on the Y axis at
// fusion_variants/2D_D_exp_fused_fft_cgemm_ifft/fused_trunc_2D.cu:165), which then runs along X. The result is the same
// truncated 2D transform pair as the reference's order (strided X axis first, :160, :170): the 2D transform is
// separable. A block owns ROWS consecutive rows of one image: its lane groups transform them in batches (one L-lane
// group per row, as in stride_DY_kernel), the 64 x ROWS tile of kept modes goes through LDS and is written / read as
// runs of ROWS * 8 contiguous bytes per mode.
#include "group_fft.h"
#include "kernels.h"

namespace tfno {

template <int LOGDY> struct GeoRows {
    using G = Geo1D<LOGDY>;
    static constexpr int BATCHES = LOGDY == 7 ? 1 : LOGDY == 8 ? 2 : LOGDY == 9 ? 4 : 8;   // rows are transformed GROUPS at a time
    static constexpr int ROWS = BATCHES * G::GROUPS;                  // rows of the image per block: 32 at every length
    static constexpr int PT = ROWS + 1;                               // pitch (complex) of the tile [64][ROWS]
    static constexpr size_t LDS_BYTES = sizeof(float2) * (size_t)(G::GROUPS * G::EXCH + 64 * PT);
};

// The forward kernel is persistent: a block walks the row blocks blockIdx.x, + gridDim.x, ... and requests the first rows
// of its next row block while it still works on the current one (x is streamed past the caches: it is read once).
template <int LOGDY>
__global__ __launch_bounds__(256) void fft_rows_trunc_kernel(const float2* __restrict__ in, float2* __restrict__ out, int DX,
                                                            long nblocks)
{
    using G = Geo1D<LOGDY>;
    using R = GeoRows<LOGDY>;
    constexpr int DY = G::DY, L = G::L, GROUPS = G::GROUPS, MM = G::MM, ROWS = R::ROWS, PT = R::PT;
    extern __shared__ float2 lds[];
    const int tid = threadIdx.x, g = tid / L, t = tid % L;
    float2* exch = lds + g * G::EXCH;
    float2* tile = lds + GROUPS * G::EXCH;

    cpx tw[16], v[16];
    load_lane_twiddles<LOGDY>(t, tw);
    // row block `blk` is rows [blk * ROWS, + ROWS) of the array of all rows of all images (DX is a multiple of ROWS)
    auto fetch = [&](long blk, int b) {
        const float2* src = in + ((blk * ROWS + b * GROUPS + g) * (long)DY) + t;
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = load_streaming(src + L * i);
    };
    long blk = blockIdx.x;
    if (blk < nblocks) fetch(blk, 0);
    for (; blk < nblocks; blk += gridDim.x) {
#pragma unroll
        for (int b = 0; b < R::BATCHES; ++b) {
            cpx gg[16], o[MM];
            fwd_pass1(v, tw, gg);
            // the next batch of rows (of the next row block after the last batch) travels under the second pass
            if (b + 1 < R::BATCHES) fetch(blk, b + 1);
            else if (blk + gridDim.x < nblocks) fetch(blk + gridDim.x, 0);
            group_forward_finish<LOGDY>(gg, exch, t, o);
#pragma unroll
            for (int a = 0; a < MM; ++a) tile[forward_mode_of_lane<LOGDY>(t, a) * PT + b * GROUPS + g] = o[a];
        }
        __syncthreads();
        const long row0 = blk * ROWS;
        float2* dst = out + (row0 / DX) * 64 * DX + row0 % DX;
#pragma unroll
        for (int i = tid; i < 64 * ROWS; i += 256) dst[(long)(i / ROWS) * DX + i % ROWS] = tile[(i / ROWS) * PT + i % ROWS];
        __syncthreads();                                         // the tile is free for the next row block
    }
}

// One block per row block, not persistent: a persistent version with the next tile requested ahead was 8-17 % slower
// (its blocks drift into lockstep and the stores arrive in bursts; the hardware's own block scheduling keeps them apart).
template <int LOGDY>
__global__ __launch_bounds__(256) void ifft_rows_pad_kernel(const float2* __restrict__ in, float2* __restrict__ out, int DX)
{
    using G = Geo1D<LOGDY>;
    using R = GeoRows<LOGDY>;
    constexpr int DY = G::DY, L = G::L, GROUPS = G::GROUPS, MM = G::MM, ROWS = R::ROWS, PT = R::PT;
    extern __shared__ float2 lds[];
    const int tid = threadIdx.x, g = tid / L, t = tid % L;
    float2* exch = lds + g * G::EXCH;
    float2* tile = lds + GROUPS * G::EXCH;
    const long row0 = (long)blockIdx.x * ROWS;                   // first of this block's rows, counted over all images

    const float2* src = in + (row0 / DX) * 64 * DX + row0 % DX;
#pragma unroll
    for (int i = tid; i < 64 * ROWS; i += 256) tile[(i / ROWS) * PT + i % ROWS] = src[(long)(i / ROWS) * DX + i % ROWS];
    cpx tw[16];
    load_lane_twiddles<LOGDY>(t, tw);
    __syncthreads();
    float2* dst = out + ((row0 + g) * (long)DY) + t;
#pragma unroll
    for (int b = 0; b < R::BATCHES; ++b) {
        cpx c[MM], yv[16];
#pragma unroll
        for (int a = 0; a < MM; ++a) c[a] = tile[(t + L * a) * PT + b * GROUPS + g];
        group_backward<LOGDY>(c, tw, exch, t, yv);
        store_row16<L, false>(dst, yv);
        dst += (long)GROUPS * DY;
    }
}

template <int LOGDY, bool INVERSE>
static hipError_t launch_rows_t(const float2* in, float2* out, int DX, long nimg, hipStream_t stream)
{
    using R = GeoRows<LOGDY>;
    static_assert(R::LDS_BYTES <= 64 * 1024, "fits the default dynamic LDS limit");
    if (DX % R::ROWS) return hipErrorInvalidValue;
    const long blocks = nimg * (DX / R::ROWS);
    if (blocks <= 0 || blocks > 0x7fffffffL) return hipErrorInvalidValue;
    if constexpr (INVERSE) {
        hipLaunchKernelGGL((ifft_rows_pad_kernel<LOGDY>), dim3((unsigned)blocks), dim3(256), R::LDS_BYTES, stream, in, out, DX);
    } else {
        // as many blocks as the CUs hold at once (LDS: 43-52 KiB per block)
        const long resident = (long)cu_count() * (long)((160 * 1024) / R::LDS_BYTES);
        hipLaunchKernelGGL((fft_rows_trunc_kernel<LOGDY>), dim3((unsigned)(blocks < resident ? blocks : resident)), dim3(256),
                           R::LDS_BYTES, stream, in, out, DX, blocks);
    }
    return hipGetLastError();
}

template <bool INVERSE>
static hipError_t launch_rows(int logDY, const float2* in, float2* out, int DX, long nimg, hipStream_t stream)
{
    switch (logDY) {
    case 7: return launch_rows_t<7, INVERSE>(in, out, DX, nimg, stream);
    case 8: return launch_rows_t<8, INVERSE>(in, out, DX, nimg, stream);
    case 9: return launch_rows_t<9, INVERSE>(in, out, DX, nimg, stream);
    case 10: return launch_rows_t<10, INVERSE>(in, out, DX, nimg, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_fft_rows_trunc(int logDY, const float2* in, float2* out, int DX, long nimg, hipStream_t stream)
{
    return launch_rows<false>(logDY, in, out, DX, nimg, stream);
}

hipError_t launch_ifft_rows_pad(int logDY, const float2* in, float2* out, int DX, long nimg, hipStream_t stream)
{
    return launch_rows<true>(logDY, in, out, DX, nimg, stream);
}

}  // namespace tfno
