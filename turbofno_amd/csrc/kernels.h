// Internal launcher declarations shared between the kernel translation units and the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>

namespace tfno {

// LDS layout of a real-expanded W' tile for v_mfma_f32_16x16x4_f32 (the block-per-item matrix-core
// 1D kernels): float index  (k/4)*kWGroup + ((k&3)>>1)*kWHalf + n'*4 + (k&1)*2 + c  holds W'[n' = 2n + c'][2k + c],
// {Wr, -Wi} for c' = 0 and {Wi, Wr} for c' = 1. An operand read (16 n' x 4 channels) takes 256 contiguous bytes per
// half wavefront: conflict free. The strides are 512 + 4 and 1024 + 8 floats so that the tile BUILD, whose lanes run
// along k (the contiguous direction of W in memory), spreads a half wavefront over all 64 banks as well; with the
// unpadded strides every lane of such a store fell on the same two banks.
constexpr int kWHalf = 516;
constexpr int kWGroup = 1032;

#ifdef __HIPCC__
// Block -> (signal set s, output tile) for the fused 1D kernels. Consecutive workgroups go to different XCDs (eight L2s),
// and every output tile of a signal set re-reads the same K input rows: the tiles of one s are therefore given block
// ids eight apart, which lands them on the same XCD at about the same time, so only the first of them reads x from
// HBM. Groups of eight signal sets are laid out as [tile][s % 8]; a tail of fewer than eight sets is laid out plainly.
//
// With that layout XCD j only ever touches the signal sets s = j mod 8, i.e. the addresses j * 8 * DY + 64 * DY * i
// within every channel row. When the channel stride S * DY * 8 bytes is a multiple of 4 MiB (batch sizes that are powers
// of two), all K + N rows of a signal set also fall on the same memory channels, and each XCD is left talking to a
// fixed part of the memory system: such grids ran 5-25 % below their neighbours (DY = 256, K = 8: S = 2048 0.53 of the
// HBM peak, S = 4096 0.61, S = 3584 0.70). For these strides XCD j walks the j-th eighth of the signal sets instead
// (tiles of a signal set on consecutive blocks of that XCD): S = 2048 0.65, S = 4096 0.71; up to -26 % at DY = 512.
// Up to a stride of 16 MiB; beyond it the grids are large enough to hide the effect and the contiguous walk costs 2-5 %.
// Only for launches that stream x from and y to HBM (`streamed`). As the middle stage of a 2D pipeline the kernel itself
// is faster in that order as well (16 images of 512 x 512, X axis first: 100 -> 94 us, half the tag and write stalls in
// L2 at the same hit rate), but the backward kernel that follows loses twice as much (472 -> 487 us): it reads the
// intermediate in its own order and finds less of it still in the Infinity Cache when the eighths were written side by
// side (its read latency at the memory side rises from 1880 to 2000 cycles, the request counts stay the same). The
// layer is what counts, so the middle stage keeps the interleaved order. (-DTFNO_MIDDLE_STAGE_WALKS_EIGHTHS builds the
// other order for measurements.)
// Workgroup b of a one-dimensional grid runs on XCD b mod 8: renumbered like this, XCD j takes the j-th eighth of n
// work items, in order, instead of every eighth item.
__device__ __forceinline__ long xcd_contiguous(long b, long n) { return (n & 7) == 0 ? (b & 7) * (n >> 3) + (b >> 3) : b; }
__host__ __device__ __forceinline__ bool xcd_walks_an_eighth_1d(long S, int DY)
{
    const long stride = S * DY * 8;
    return stride % (4L << 20) == 0 && stride <= (16L << 20);      // S is then a multiple of 8
}
__device__ __forceinline__ void decode_block_1d(long S, int ntiles, int DY, bool streamed, long& s, int& tile)
{
#ifdef TFNO_MIDDLE_STAGE_WALKS_EIGHTHS
    streamed = true;
#endif
    if (streamed && xcd_walks_an_eighth_1d(S, DY)) {
        const long id = blockIdx.x, q = id >> 3;
        s = (id & 7) * (S / 8) + q / ntiles;
        tile = (int)(q % ntiles);
        return;
    }
    const long id = blockIdx.x, full = (S / 8) * 8;
    if (id < full * ntiles) {
        const long grp = id / (8 * ntiles);
        const int rem = (int)(id % (8 * ntiles));
        tile = rem / 8;
        s = grp * 8 + rem % 8;
    } else {
        const long rem = id - full * ntiles;
        s = full + rem / ntiles;
        tile = (int)(rem % ntiles);
    }
}
#endif

// Share of the work of a pair of persistent blocks (2p on an even XCD, 2p + 1 on an odd one) that the even block takes in
// the store-bound backward kernels, in parts of kEvenShareDen: 17 on MI355X (gfx950, 8 XCDs of 32 CUs), whose odd XCDs
// sustain about a fifth less store traffic than the even ones (measured; 17 and 18 level, 19 worse); an even 16 on any
// other part or partition, where neither that ratio nor "block parity = XCD parity" is known to hold. A kernel argument,
// resolved per device by even_share_parts().
constexpr int kEvenShareDen = 32;
int even_share_parts();

// compute units of the current device (cached per device)
int cu_count();

// Kernels with more than 64 KiB of dynamic LDS need hipFuncAttributeMaxDynamicSharedMemorySize raised once per device.
// `done` is the kernel's own bit mask of devices already served (one static per launcher); safe from several threads:
// a second caller at worst repeats the idempotent call.
inline hipError_t allow_dynamic_lds(const void* kernel, size_t bytes, std::atomic<unsigned long long>& done)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const unsigned long long bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    return e;
}

// 1D fused layer / Y stage of the three-kernel 2D pipeline. S = number of signals per channel.
// algo: 0 = chosen by size, 1 ... 8 = one of the kernels below (include/turbofno.h, turbofno_set_1d_algo).
hipError_t launch_fused_fft_cgemm_ifft(int logDY, long S, int N, int K, const float2* x, const float2* W, float2* y,
                                       float2 alpha, int algo, hipStream_t stream, bool y_is_reread = false);
// The kernel that call runs (the selector values 1 ... 8), from the sizes alone.
enum {
    kFused1dSimt = 1, kFused1dMfma512 = 2, kFused1dMfma256 = 3, kFused1dMfma512Tile32 = 4, kFused1dWave = 5,
    kFused1dSplit = 6, kFused1dCluster = 7, kFused1dWide = 8
};
int pick_fused_1d_kernel(int logDY, long S, int N, int K, int algo, bool keep_y, long cus, bool exchange_attached);

// Cluster variant of the fused 1D layer (layer1d_cluster.hip): cluster size for a problem on `cus` compute units (0 = not
// applicable), the launch (hipErrorNotReady when no exchange buffer is attached to the stream), the bound of its
// inter-block waits in ticks of the 100 MHz wall clock, and the registry of caller-owned exchange buffers.
int cluster_size_1d(int logDY, long S, int N, int K, long cus);
hipError_t launch_fused_cluster(long S, int N, int K, int P, const float2* x, const float2* W, float2* y, float2 alpha,
                                hipStream_t stream);
void set_cluster_wait_ticks(unsigned long long ticks);
size_t exchange_bytes(long cus);                                    // cus <= 0: the current device
hipError_t exchange_attach(hipStream_t stream, void* buffer, size_t bytes);   // null buffer: detach
bool exchange_attached(hipStream_t stream);
hipError_t exchange_gave_up(hipStream_t stream, unsigned* count);   // waits for the stream

// Large grids, DY = 128 / 256 (layer1d_wide.hip): one block per (signal set, 128 or 64 output channels), three-real-product
// contraction.
hipError_t launch_fused_wide(int logDY, long S, int N, int K, const float2* x, const float2* W, float2* y, float2 alpha,
                             hipStream_t stream, int keep_y = 0);

// Halves of the fused kernel (variants B and C) and the stand-alone contiguous transforms (variant A).
hipError_t launch_fused_fft_cgemm(int logDY, long S, int N, int K, const float2* x, const float2* W, float2* C,
                                  float2 alpha, float2 beta, hipStream_t stream);
hipError_t launch_fused_cgemm_ifft(int logDY, long S, int N, int K, const float2* A, const float2* W, float2* y,
                                   float2 alpha, hipStream_t stream);
hipError_t launch_fft_stride_DY(int logDY, const float2* in, float2* out, long nsig, hipStream_t stream);
hipError_t launch_ifft_stride_DY(int logDY, const float2* in, float2* out, long nsig, hipStream_t stream);

// X-axis (element stride DY) truncated forward / zero-padded backward transforms.
hipError_t launch_fft_stride(int logDX, const float2* in, float2* out, int DY, long nsig, hipStream_t stream);
hipError_t launch_ifft_stride(int logDX, const float2* in, float2* out, int DY, long nsig, hipStream_t stream);

// Y-axis (contiguous) transforms of the rows-first 2D pipeline (rows_fft.hip): in[img][DX][DY] -> out[img][64][DX] and
// back; the intermediates are transposed so that the fused 1D kernel runs along X on them.
hipError_t launch_fft_rows_trunc(int logDY, const float2* in, float2* out, int DX, long nimg, hipStream_t stream);
hipError_t launch_ifft_rows_pad(int logDY, const float2* in, float2* out, int DX, long nimg, hipStream_t stream);

// Whole-image 2D path (DY in {128, 256}; DX in {128, 256}, or 512 / 1024 as two / four decimated parts of 256 rows):
// truncated 2D forward transform per image, mode-space CGEMM on the matrix cores, zero-padded 2D backward transform per
// image. nimg: whole images; the C ABI rejects counts beyond INT_MAX. With R = DX / 256 > 1 parts, launch_fft2d_trunc
// writes R * nimg spectra of 4096 modes (part r of image i at index r * nimg + i), to be summed over r: the contraction
// does that when the parts are its channels r * K + k (launch_cgemm_modes with K = R * channels and w_period = channels);
// launch_ifft2d_pad reads nimg spectra.
hipError_t launch_fft2d_trunc(int logDX, int logDY, const float2* x, float2* spec, int nimg, hipStream_t stream);
hipError_t launch_ifft2d_pad(int logDX, int logDY, const float2* spec, float2* y, int nimg, hipStream_t stream);
hipError_t launch_cgemm_modes(const float2* A, const float2* W, float2* C, long Mtot, int N, int K, float2 alpha,
                              float2 beta, hipStream_t stream, int w_period = 0);

}  // namespace tfno
