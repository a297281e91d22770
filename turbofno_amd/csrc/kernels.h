// Internal launcher declarations shared between the kernel translation units and the C ABI.
#pragma once
#include <hip/hip_runtime.h>

namespace tfno {

// compute units of the current device (cached)
int cu_count();

// 1D fused layer / Y stage of the three-kernel 2D pipeline. S = number of signals per channel.
// algo: 0 = chosen by size, 1 = SIMT contraction, 2 = contraction on the matrix cores.
hipError_t launch_fused_fft_cgemm_ifft(int logDY, long S, int N, int K, const float2* x, const float2* W, float2* y,
                                       float2 alpha, int algo, hipStream_t stream);

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

// Whole-image 2D path (DX, DY in {128, 256}): truncated 2D forward transform per image, mode-space CGEMM
// on the matrix cores, zero-padded 2D backward transform per image.
hipError_t launch_fft2d_trunc(int logDX, int logDY, const float2* x, float2* spec, long nimg, hipStream_t stream);
hipError_t launch_ifft2d_pad(int logDX, int logDY, const float2* spec, float2* y, long nimg, hipStream_t stream);
hipError_t launch_cgemm_modes(const float2* A, const float2* W, float2* C, long Mtot, int N, int K, float2 alpha,
                              float2 beta, hipStream_t stream);

}  // namespace tfno
