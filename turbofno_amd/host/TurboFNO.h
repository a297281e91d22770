// Tunables of the host drivers. Mirrors the role of the reference's utils/TurboFNO.h:2-20 (the GEMM tile
// height, which is also the number of retained modes per axis, the K granularity, and the globals
// ntest / threadblock_bs). The reference's warp-level tile constants have no counterpart here: the
// gfx950 kernels fix their own wave64 tiling at compile time.
#pragma once

#define THREADBLOCK_M 64      // retained modes per transformed axis = rows one signal contributes to the GEMM
#define THREADBLOCK_K 8       // K (input channels) must be a multiple of this

extern int ntest;             // timed iterations per problem (reference default 5)
extern int threadblock_bs;    // columns per block argument of the X-axis kernels (kept for signature parity)
