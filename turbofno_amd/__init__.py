"""turbofno_amd -- MI355X (gfx950) implementation of TurboFNO's fused spectral layer.

The product is libturbofno.so (hand-written HIP kernels behind the C ABI of include/turbofno.h) and
the C++ drivers under turbofno_amd/host. This module is the thin Python binding used by the tests
and the benchmark: torch supplies device memory and streams, nothing else. There is no CPU or
library fallback: if the shared library is missing, importing `turbofno_amd.api` raises.
"""
from .api import (  # noqa: F401
    MODES,
    ExchangeBuffer,
    TurboFNOError,
    cgemm,
    exchange_bytes,
    fft2d_trunc,
    ifft2d_pad,
    fft_stride,
    fft_stride_DY,
    fused_cgemm_ifft,
    fused_fft_cgemm,
    fused_fft_cgemm_ifft,
    ifft_stride,
    ifft_stride_DY,
    layer_1d,
    layer_2d,
    layer_2d_noalloc,
    layer_2d_workspace_bytes,
    lib,
    library_path,
    query_1d_kernel,
    query_2d_algo,
    set_1d_algo,
    set_exchange_wait_us,
)

ALGO_AUTO, ALGO_THREE_KERNEL, ALGO_WHOLE_IMAGE, ALGO_ROWS_FIRST = 0, 1, 2, 3
