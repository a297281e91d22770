#!/usr/bin/env python3
"""Writes the golden vectors of tests/golden/ (run from the repository root: python tests/golden/make_golden.py).

The reference holds no test vectors for the fused spectral layer and cannot be built or run, so these vectors come
from an independent library evaluation of the frozen definition: numpy.fft (pocketfft) in float64, in the
"mix channels in space, then low-pass" order, which shares no code and no evaluation order with the oracle
(oracle/turbofno_oracle.c) or the kernels:

    y[n] = ifft_unnormalised( keep64( fft( alpha * sum_k W[k][n] x[k] ) ) )

Inputs are regenerated in the tests from the seeds stored next to the outputs (numpy default_rng streams are stable
across numpy versions); only the expected outputs are stored, subsampled for the 2D case to keep the files small.
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def inputs_1d(seed, bs, DY, K, N):
    rng = np.random.default_rng(seed)
    x = (rng.uniform(-1, 1, (K, bs, DY)) + 1j * rng.uniform(-1, 1, (K, bs, DY))).astype(np.complex64)
    W = ((rng.uniform(-1, 1, (N, K)) + 1j * rng.uniform(-1, 1, (N, K))) / np.sqrt(K)).astype(np.complex64)
    return x, W


def inputs_2d(seed, bs, DX, DY, K, N):
    rng = np.random.default_rng(seed)
    x = (rng.uniform(-1, 1, (K, bs, DX, DY)) + 1j * rng.uniform(-1, 1, (K, bs, DX, DY))).astype(np.complex64)
    W = ((rng.uniform(-1, 1, (N, K)) + 1j * rng.uniform(-1, 1, (N, K))) / np.sqrt(K)).astype(np.complex64)
    return x, W


def expected_1d(x, W, alpha):
    mixed = alpha * np.einsum("nk,ksj->nsj", W.astype(np.complex128), x.astype(np.complex128))
    spec = np.fft.fft(mixed, axis=-1)
    spec[..., 64:] = 0
    return np.fft.ifft(spec, axis=-1) * x.shape[-1]


def expected_2d(x, W, alpha, channels):
    Wc = W.astype(np.complex128)[channels]
    mixed = alpha * np.einsum("nk,kbxy->nbxy", Wc, x.astype(np.complex128))
    spec = np.fft.fft2(mixed, axes=(-2, -1))
    spec[..., 64:, :] = 0
    spec[..., :, 64:] = 0
    return np.fft.ifft2(spec, axes=(-2, -1)) * (x.shape[-2] * x.shape[-1])


CASES_1D = {   # name: (seed, bs, DY, K, N, alpha, stored output channels)
    "config1_bs1_DY128_K8_N64": (101, 1, 128, 8, 64, 1.0 + 0.0j, tuple(range(64))),
    "bs3_DY256_K24_N128_alpha": (102, 3, 256, 24, 128, 1.0 - 1.0j, (0, 64, 127)),
    "bs2_DY1024_K8_N64": (103, 2, 1024, 8, 64, 1.0 + 0.0j, (1, 62)),
}
CASES_2D = {   # name: (seed, bs, DX, DY, K, N, alpha, channels, stride)
    "bs1_128x128_K16_N64": (201, 1, 128, 128, 16, 64, 1.0 + 0.0j, (0, 17, 63), 4),
    "bs2_256x128_K8_N64_alpha": (202, 2, 256, 128, 8, 64, 1.0 - 1.0j, (5, 40), 8),
}


def main():
    out = {}
    for name, (seed, bs, DY, K, N, alpha, ch) in CASES_1D.items():
        x, W = inputs_1d(seed, bs, DY, K, N)
        out["1d/" + name] = expected_1d(x, W, alpha)[list(ch)].astype(np.complex64)
    for name, (seed, bs, DX, DY, K, N, alpha, ch, st) in CASES_2D.items():
        x, W = inputs_2d(seed, bs, DX, DY, K, N)
        out["2d/" + name] = expected_2d(x, W, alpha, list(ch))[..., ::st, ::st].astype(np.complex64)
    np.savez(os.path.join(HERE, "layer_outputs.npz"), **out)
    for k, v in out.items():
        print(k, v.shape)


if __name__ == "__main__":
    main()
