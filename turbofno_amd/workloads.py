"""Seeded synthetic inputs for the five benchmark configurations (numpy, complex64).

Layouts are the kernels' own: x[K][bs*dimX][DY] (1D) or x[K][bs][DX][DY] (2D), W[N][K] with element
W[k + n*K]. Distributions follow the configuration list of the build's baseline description.
"""
import numpy as np


def _uniform_c64(rng, shape):
    return (rng.uniform(-1.0, 1.0, shape) + 1j * rng.uniform(-1.0, 1.0, shape)).astype(np.complex64)


def weights_uniform(rng, N, K):
    return (_uniform_c64(rng, (N, K)) / np.sqrt(K)).astype(np.complex64)


def weights_normal(rng, N, K):
    return ((rng.standard_normal((N, K)) + 1j * rng.standard_normal((N, K))) / np.sqrt(K)).astype(np.complex64)


def uniform_1d(seed, bs, DY, K, N, dimX=1):
    """configs 1 and 2: re/im i.i.d. uniform[-1,1], weights uniform / sqrt(K)."""
    rng = np.random.default_rng(seed)
    return _uniform_c64(rng, (K, bs * dimX, DY)), weights_uniform(rng, N, K)


def smooth_1d(seed, bs, DY, K, N):
    """config 3: sum of 8 random-phase sinusoids at frequencies 1..32 plus 0.01 N(0,1) noise per channel."""
    rng = np.random.default_rng(seed)
    j = np.arange(DY)

    def part():
        f = rng.integers(1, 33, size=(K, bs, 8, 1))
        ph = rng.uniform(0, 2 * np.pi, size=(K, bs, 8, 1))
        return np.sin(2 * np.pi * f * j / DY + ph).sum(axis=2) + 0.01 * rng.standard_normal((K, bs, DY))

    x = (part() + 1j * part()).astype(np.complex64)
    return x, weights_uniform(rng, N, K)


def uniform_2d(seed, bs, DX, DY, K, N):
    """config 4: re/im i.i.d. uniform[-1,1]."""
    rng = np.random.default_rng(seed)
    return _uniform_c64(rng, (K, bs, DX, DY)), weights_uniform(rng, N, K)


def vorticity_2d(seed, bs, DX, DY, K, N):
    """config 5 (headline): Gaussian random field with power spectrum (|k|^2 + 9)^-2.5, unit variance per
    channel; complex normal weights / sqrt(K)."""
    rng = np.random.default_rng(seed)
    kx = np.fft.fftfreq(DX, 1.0 / DX)[:, None]
    ky = np.fft.fftfreq(DY, 1.0 / DY)[None, :]
    amp = (kx * kx + ky * ky + 9.0) ** -1.25
    x = np.empty((K, bs, DX, DY), dtype=np.complex64)
    for k in range(K):
        white = rng.standard_normal((bs, DX, DY)) + 1j * rng.standard_normal((bs, DX, DY))
        field = np.fft.ifft2(white * amp, axes=(-2, -1))
        field /= np.sqrt(np.mean(np.abs(field) ** 2))
        x[k] = field.astype(np.complex64)
    return x, weights_normal(rng, N, K)
