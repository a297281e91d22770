// Seeded synthetic inputs of the five benchmark configurations, in the kernels' own layouts
// (x[K][bs*dimX][DY] or x[K][bs][DX][DY], W[k + n*K]; interleaved complex64). The reference's mains know one input
// only, +-{0..9}e-3 from rand() (utils/utils.cu:37-43, fused.cu:61-62); these are the distributions the benchmark
// configurations name instead, drawn from std::mt19937_64 so that a (kind, seed) pair always gives the same data:
//   uniform    re / im i.i.d. uniform[-1, 1]; weights uniform[-1, 1] / sqrt(K)              (configurations 1, 2, 4)
//   smooth     per channel and signal: sum of 8 sinusoids, frequencies uniform in {1..32}, phases uniform in [0, 2 pi),
//              plus 0.01 N(0,1) (real and imaginary part drawn independently); weights as above   (configuration 3)
//   vorticity  2D Gaussian random field per image: white complex N(0,1) spectrum times (|k|^2 + 9)^-1.25, inverse 2D
//              transform, scaled to unit variance per channel; weights complex N(0,1) / sqrt(K)  (configuration 5)
// The drivers select them with TURBOFNO_INPUTS=uniform|smooth|vorticity (default: the reference's rand() fill) and
// TURBOFNO_SEED (default 0x5EED + the configuration's number).
#pragma once
#include <cstddef>
#include <cstdint>
#include <vector>

enum class InputKind { reference_rand, uniform, smooth, vorticity };

// "uniform" / "smooth" / "vorticity" -> kind; anything else (or null) -> reference_rand
InputKind input_kind_from_name(const char* name);
uint64_t default_seed(InputKind kind);

// x: channels * signals * DY complex values (2D: signals = bs * DX rows of DY samples; `dx` = DX, 0 for 1D inputs).
// Returns interleaved (re, im) floats.
std::vector<float> generate_inputs(InputKind kind, uint64_t seed, int channels, long signals_per_channel, int dx, int dy);
// W[k + n*K], K contiguous
std::vector<float> generate_weights(InputKind kind, uint64_t seed, int K, int N);
