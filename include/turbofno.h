/*
 * turbofno.h -- C ABI of the MI355X (gfx950) implementation of TurboFNO's fused spectral layer
 * (variant D, 1D and 2D): forward C2C FFT -> keep the 64 lowest modes -> complex GEMM over the
 * channel dimension -> zero-pad -> backward FFT.
 *
 * The reference has no library API; its boundary is "host main() launches a __global__ kernel picked
 * from a table indexed by log2(len)-7". Each entry point below replaces one such table entry and
 * keeps its argument meaning. Reference paths are relative to the TurboFNO checkout.
 *
 * Conventions
 *   - All data pointers are DEVICE pointers to complex64 (interleaved float re, im). The caller owns
 *     every buffer, including the 2D workspace and the optional exchange buffer of clustered launches;
 *     no entry point allocates or frees memory, on the device or pinned on the host.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream). Calls are asynchronous and
 *     never synchronise, with one documented exception: turbofno_exchange_status waits for its stream.
 *   - Return value 0 = success; otherwise a TURBOFNO_ERR_* code, with a human-readable explanation
 *     available from turbofno_last_error_string() (thread local). The library never exits the process
 *     (the reference exits from its mains via CHECK_CUDA_KERNEL, utils/utils.cuh:17-25).
 *   - 64 modes are retained per transformed axis (fused.cu:105, README.md:90); forward transforms use
 *     exp(-2 pi i jm/D), backward transforms exp(+2 pi i jm/D) and are UNNORMALISED.
 *   - Layouts: x[K][S][DY] (signal (k,s) at (k*S+s)*DY), W[k + n*K], y[N][S][DY]; in 2D
 *     x[K][bs][DX][DY], y[N][bs][DX][DY].
 */
#ifndef TURBOFNO_H
#define TURBOFNO_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TURBOFNO_OK               0
#define TURBOFNO_ERR_INVALID_ARG  1  /* null pointer, non-positive size, K % 8, N % 64, M % 64 ...      */
#define TURBOFNO_ERR_UNSUPPORTED  2  /* transform length outside the built set                           */
#define TURBOFNO_ERR_WORKSPACE    3  /* workspace missing or too small                                   */
#define TURBOFNO_ERR_HIP          4  /* the HIP runtime reported a launch error                          */
#define TURBOFNO_ERR_EXCHANGE     5  /* turbofno_exchange_status only: cluster members ran out of their wait (results valid, launches slow) */

#define TURBOFNO_MODES 64

/* algorithms of turbofno_layer_2d */
#define TURBOFNO_2D_AUTO          0
#define TURBOFNO_2D_THREE_KERNEL  1  /* X transform, fused Y stage, X inverse: the reference's structure */
#define TURBOFNO_2D_WHOLE_IMAGE   2  /* one block per image + matrix-core CGEMM                          */
#define TURBOFNO_2D_ROWS_FIRST    3  /* Y transform of whole rows, fused X stage, Y inverse of whole rows */

/*
 * Fused 1D layer kernel. Replaces the table entries fused_fft_cgemm_ifft[log2(DY)-7]
 *   fusion_variants/1D_D_exp_fused_fft_cgemm_ifft/fused.cu:15-16 (table), :119-126 (launch)
 *   fusion_variants/1D_D_exp_fused_fft_cgemm_ifft/fused_fft_cgemm_ifft_7.cuh:9 (signature
 *   (int M, int N, int K, float2* FFT_input, float2* B, float2* C, float2* FFT_output, float2 alpha, float2 beta))
 * M = 64 * S where S = bs*dimX signals per channel. `C` is unused by the reference kernel (its beta*C
 * term is commented out, fused_fft_cgemm_ifft_7.cuh:186-187) and may be NULL; beta is ignored.
 * Requires logDY in {7, 8, 9, 10}, M % 64 == 0, N % 64 == 0, K % 8 == 0 (utils/TurboFNO.h:2-4).
 * On small grids with K >= 64 this entry point and turbofno_layer_1d use the exchange buffer of the stream when the
 * caller has attached one: see "Clustered launches" below.
 */
int turbofno_fused_fft_cgemm_ifft(int logDY, long M, int N, int K, const void* x, const void* W, void* C, void* y,
                                  float alpha_re, float alpha_im, float beta_re, float beta_im, void* stream);

/*
 * X-axis stage kernels of the 2D pipeline. Replace the table entries fft_stride[log2(DX)-7] and
 * ifft_stride[log2(DX)-7], signature (float2* in, float2* out, int threadblock_bs, int DY, int total, int dimX):
 *   fusion_variants/2D_D_exp_fused_fft_cgemm_ifft/fused_trunc_2D.cu:27-28 (tables), :153-160, :170 (launches)
 * forward : in[total/DY][DX][DY] -> out[total/DY][dimX][DY]   FFT along DX, first dimX rows kept
 * backward: in[total/DY][dimX][DY] -> out[total/DY][DX][DY]   rows >= dimX taken as zero, backward FFT along DX
 * `total` = number of columns (DY * channels * bs). threadblock_bs (columns per block in the
 * reference) is accepted for signature compatibility and ignored. Requires logDX in {7, 8, 9, 10},
 * dimX == 64, DY % 16 == 0, total % DY == 0.
 */
int turbofno_fft_stride(int logDX, const void* in, void* out, int threadblock_bs, int DY, long total, int dimX,
                        void* stream);
int turbofno_ifft_stride(int logDX, const void* in, void* out, int threadblock_bs, int DY, long total, int dimX,
                         void* stream);

/*
 * Whole 1D layer, as run by TurboFNO_1D_D for one (bs, dimX, DY, N, K) problem
 * (fusion_variants/1D_D_exp_fused_fft_cgemm_ifft/fused.cu:104-126). One kernel launch.
 */
int turbofno_layer_1d(int bs, int dimX, int DY, int K, int N, const void* x, const void* W, void* y,
                      float alpha_re, float alpha_im, void* stream);

/*
 * Whole 2D layer, as run by TurboFNO_2D_D for one (bs, DX, DY, N, K) problem
 * (fusion_variants/2D_D_exp_fused_fft_cgemm_ifft/fused_trunc_2D.cu:133-172). The reference keeps its
 * intermediates t1/t2 in buffers owned by main(); here the caller passes `workspace` of at least
 * turbofno_layer_2d_workspace_bytes(...) bytes (256-byte aligned). x is not modified.
 * algo: TURBOFNO_2D_AUTO picks by size (lengths up to 256: WHOLE_IMAGE from a batch of 8, and from a batch of 4 when
 * there are enough images; THREE_KERNEL below; longer axes: WHOLE_IMAGE from 0.6 to 4.5 GiB of input and output,
 * depending on the lengths, else ROWS_FIRST or THREE_KERNEL); the workspace query with the same arguments,
 * and turbofno_query_2d_algo, make the same
 * choice. Every algorithm takes every pair of lengths in {128, 256, 512, 1024} (WHOLE_IMAGE handles images of 512 or
 * 1024 rows as two or four interleaved parts of 256 rows that the contraction sums over). ROWS_FIRST is the three-stage structure with the axes exchanged
 * (the contiguous axis is transformed first and last, so that x and y move as whole rows): same result, the 2D
 * transform being separable; its intermediates are [images][64][DX].
 */
size_t turbofno_layer_2d_workspace_bytes(int bs, int DX, int DY, int K, int N, int algo);
int turbofno_layer_2d(int bs, int DX, int DY, int K, int N, const void* x, const void* W, void* y,
                      float alpha_re, float alpha_im, void* workspace, size_t workspace_bytes, int algo, void* stream);

/*
 * Stages of the whole-image 2D algorithm, exposed so that they can be timed, profiled and composed
 * individually (the reference's variants A/B/C compose the same layer from separately launched stages).
 *   turbofno_fft2d_trunc : x[nimg][DX][DY] -> spec[nimg][4096]  truncated 2D forward transform per image
 *   turbofno_ifft2d_pad  : spec[nimg][4096] -> y[nimg][DX][DY]  zero-padded 2D backward transform per image
 * The 4096 retained modes of an image are stored in an order private to these two kernels (element
 * mm*(4*DX) + q*(DX/16) + t holds mode (p = t + (DX/16)*mm, q)); a GEMM over the channel dimension does
 * not care. Requires DX in {128, 256} and DY in {128, 256, 512, 1024} (the layer handles longer DX as interleaved
 * parts, which have no stand-alone meaning).
 *   turbofno_cgemm : C[m + n*M] = alpha * sum_k A[m + k*M] * B[k + n*K] + beta * C[m + n*M] (column major,
 *   lda = M, ldb = K, ldc = M) on the fp32 matrix cores. Replaces the reference's cgemm kernel
 *   (fusion_variants/1D_A_exp_fft+cgemm+ifft/cgemm.cuh:4, launch 1D_A.../fused.cu:199), same argument order
 *   (M, N, K, A, B, C, alpha, beta). C is read only when beta != 0. Requires M % 64 == 0, M < 2^27,
 *   N % 64 == 0, K % 8 == 0.
 */
int turbofno_fft2d_trunc(int DX, int DY, const void* x, void* spec, long nimg, void* stream);
int turbofno_ifft2d_pad(int DX, int DY, const void* spec, void* y, long nimg, void* stream);
int turbofno_cgemm(long M, int N, int K, const void* A, const void* B, void* C, float alpha_re, float alpha_im,
                   float beta_re, float beta_im, void* stream);

/*
 * Stages of the unfused and half-fused variants (A, B, C), so that every executable of the reference's
 * ablation can be rebuilt on this library.
 *   turbofno_fft_stride_DY / turbofno_ifft_stride_DY replace the table entries fft_stride_DY[log2(DY)-7] and
 *   ifft_stride_DY[log2(DY)-7], signature (float2* in, float2* out, int threadblock_bs, int total)
 *   (fusion_variants/1D_A_exp_fft+cgemm+ifft/fused.cu:27-28 tables, :195,:203 launches):
 *     forward : in[total][DY] -> out[total][64]     backward: in[total][64] -> out[total][DY]
 *   with `total` = number of contiguous signals (dimX * channels * bs).
 *   turbofno_fused_fft_cgemm replaces fused_fft_cgemm[log2(DY)-7] of variant B
 *   (fusion_variants/1D_B_exp_fused_fft_cgemm+ifft/fused_fft_cgemm_8.cuh:8, launch 1D_B.../fused.cu:141):
 *     C[m + n*M] = alpha * sum_k FFT_trunc(x)[m + k*M] * W[k + n*K] + beta * C[m + n*M].
 *   turbofno_fused_cgemm_ifft replaces fused_cgemm_ifft[log2(DY)-7] of variant C
 *   (fusion_variants/1D_C_exp_fft+fused_cgemm_ifft/fused_cgemm_ifft_8.cuh:9, launch 1D_C.../fused.cu:144):
 *     y = iFFT_pad(alpha * A * W), A[m + k*M] column major; C and beta are unused there and here.
 * Same preconditions as turbofno_fused_fft_cgemm_ifft.
 */
int turbofno_fft_stride_DY(int logDY, const void* in, void* out, int threadblock_bs, long total, void* stream);
int turbofno_ifft_stride_DY(int logDY, const void* in, void* out, int threadblock_bs, long total, void* stream);
int turbofno_fused_fft_cgemm(int logDY, long M, int N, int K, const void* x, const void* W, void* C, float alpha_re,
                             float alpha_im, float beta_re, float beta_im, void* stream);
int turbofno_fused_cgemm_ifft(int logDY, long M, int N, int K, const void* A, const void* W, void* C, void* y,
                              float alpha_re, float alpha_im, float beta_re, float beta_im, void* stream);

/*
 * The 2D layer for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc. No counterpart in the reference (its mains allocate every buffer themselves,
 * fused_trunc_2D.cu:68-85). Same arguments and results as turbofno_layer_2d, without the workspace: the
 * intermediates live in a static device array of TURBOFNO_NOALLOC_SCRATCH_BYTES that every GPU the library runs on
 * holds until the process ends. The call allocates and frees nothing, whatever the sizes and whether or not an exchange
 * buffer is attached to the stream. `stream` must belong to the current device. Problems whose intermediates
 * (turbofno_layer_2d_workspace_bytes with the same arguments) exceed that size are refused with
 * TURBOFNO_ERR_WORKSPACE; the headline problem bs=16, 256 x 256, K=N=64 fits exactly. The first call on a device
 * resolves the array's address (make it outside any graph capture). All calls on one GPU share the one array:
 * calls that overlap on the same GPU (different streams, different threads) race; calls on one stream are ordered.
 */
#define TURBOFNO_NOALLOC_SCRATCH_BYTES (64u << 20)
int turbofno_layer_2d_noalloc(int bs, int DX, int DY, int K, int N, const void* x, const void* W, void* y,
                              float alpha_re, float alpha_im, int algo, void* stream);

/*
 * Process-wide choice of the fused 1D kernel behind turbofno_fused_fft_cgemm_ifft / turbofno_layer_1d and the Y stage
 * of the three-kernel 2D path (their reference-shaped signatures have no room for a selector): 0 = by problem size
 * (default), 1 = SIMT contraction, 2 / 3 = matrix cores with 512- / 256-thread blocks, 4 = matrix cores, 512 threads,
 * 32-channel output tiles, 5 = matrix cores, one wavefront per signal set and output tile, 6 = matrix cores, the K
 * channels of an item split over the waves of a block, 7 = matrix cores, the K channels of a signal set split over a
 * cluster of blocks (see below), 8 = matrix cores, 256-thread blocks with tiles of 128 output channels and three real
 * products per complex one (DY = 128 / 256). A value a kernel is not built for falls back to the choice by size. Meant for tests and measurements; set returns TURBOFNO_ERR_INVALID_ARG outside 0..TURBOFNO_1D_ALGO_MAX.
 */
#define TURBOFNO_1D_ALGO_MAX 8
int turbofno_set_1d_algo(int algo);
int turbofno_get_1d_algo(void);

/*
 * Clustered launches (no counterpart in the reference; opt-in). On small grids with K >= 64 (DY = 256, N = 64 or 128,
 * every block on a CU of its own: the reference's large-hidden 1D shapes) the fused 1D layer can split the K channels of
 * a signal set over 2 - 8 blocks, which exchange partial products through device memory, instead of repeating all K
 * forward transforms in every block of a signal set. That memory is the CALLER's:
 *   turbofno_exchange_bytes(cu)   size of an exchange buffer for a device of `cu` compute units (0 = the current
 *                                 device): 64 KiB + 128 B per compute unit + 256 B (16.03 MiB on 256 CUs);
 *   turbofno_exchange_attach      registers `buffer` (device memory, 256-byte aligned, at least that size) for the 1D
 *                                 layer calls on `stream` of the current device and clears its counters with a small
 *                                 kernel on that stream (no allocation, no synchronisation). Not inside a capture of that
 *                                 stream. Attaching again replaces the buffer;
 *   turbofno_exchange_detach      forgets it. Detach before freeing the buffer or destroying the stream; work already
 *                                 enqueued (or captured into a graph) keeps using the memory until it has run.
 * While a buffer is attached, turbofno_fused_fft_cgemm_ifft / turbofno_layer_1d on that stream (and the middle stage of
 * the three-stage 2D paths) take the clustered kernel where it applies by size; without one they run kernels that need
 * no exchange. Calls on one stream are ordered and share its buffer; use one buffer per stream, never one buffer on two
 * streams. A graph captured on the stream holds the buffer's address: do not replay it concurrently with other 1D
 * layer calls that use the same buffer.
 * Results do not depend on the exchange working: every inter-block wait is bounded (default 100 us,
 * turbofno_set_exchange_wait_us, process-wide; 0 = never wait: every member works alone, for tests), and a cluster
 * member that does not get the other members' partial products in time - or that starts so late that the others are
 * already publishing theirs, as can happen on the first launch after the GPU has been idle - computes their share
 * itself, so the output of every launch is valid, only later (by some 15 - 50 us, plus the wait if it came to that).
 * Such a member counts itself in the buffer:
 *   turbofno_exchange_status      WAITS for the work enqueued on `stream`, stores the count since the last call in
 *                                 *gave_up (may be NULL) and clears it; returns TURBOFNO_ERR_EXCHANGE when the count
 *                                 was not zero (advisory: the members of a cluster did not run side by side, i.e. the
 *                                 clustered kernel does not suit the way this process shares the GPU; detach the
 *                                 buffer to stop using it), TURBOFNO_OK otherwise and when no buffer is attached.
 */
size_t turbofno_exchange_bytes(int compute_units);
int turbofno_exchange_attach(void* stream, void* buffer, size_t bytes);
int turbofno_exchange_detach(void* stream);
int turbofno_exchange_status(void* stream, unsigned* gave_up);
int turbofno_set_exchange_wait_us(unsigned long long microseconds);

/*
 * What the size rules choose, as plain integer functions (no GPU work; no counterpart in the reference, whose tables
 * are indexed by log2(length) - 7 alone):
 *   turbofno_query_2d_algo    the algorithm turbofno_layer_2d(..., algo) runs for these sizes: TURBOFNO_2D_THREE_KERNEL,
 *                             _WHOLE_IMAGE or _ROWS_FIRST; 0 for arguments the layer would refuse.
 *   turbofno_query_1d_kernel  the kernel behind turbofno_fused_fft_cgemm_ifft(logDY, M, N, K, ...) under the current
 *                             turbofno_set_1d_algo selector, in that selector's numbering (1 ... 8); 0 for arguments
 *                             the call would refuse. compute_units = 0 asks the current device (the only case that
 *                             touches the HIP runtime), any other value answers for a device of that many compute
 *                             units; exchange_attached says whether the stream has an exchange buffer.
 */
int turbofno_query_2d_algo(int bs, int DX, int DY, int K, int N, int algo);
int turbofno_query_1d_kernel(int logDY, long M, int N, int K, int compute_units, int exchange_attached);

/* Explanation of the last non-zero return value on this thread ("" if none). Never NULL. */
const char* turbofno_last_error_string(void);

/* ABI version of this header (bumped on incompatible change). */
int turbofno_abi_version(void);   /* 2: exchange buffers are caller-owned; query functions */

#ifdef __cplusplus
}
#endif
#endif /* TURBOFNO_H */
