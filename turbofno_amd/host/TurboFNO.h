// Tunables of the host drivers. Mirrors the role of the reference's utils/TurboFNO.h:2-20 (tile
// constants and the globals ntest / threadblock_bs); the tile values are the ones the gfx950 kernels
// are built with, not the reference's warp-32 tiling.
#pragma once

#define THREADBLOCK_M 64      // retained modes per signal = rows of one GEMM tile
#define THREADBLOCK_N 64      // output channels per block
#define THREADBLOCK_K 8       // granularity K must be a multiple of
#define TURBOFNO_WAVE 64      // lanes per wavefront
#define THREAD_NUM 256        // threads per block of the fused 1D kernel

extern int ntest;             // timed iterations per problem (reference default 5)
extern int threadblock_bs;    // columns per block argument of the X-axis kernels (kept for signature parity)
