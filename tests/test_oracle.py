"""Pins the CPU oracle (oracle/turbofno_oracle.c) without the reference.

The reference ships no tests, golden vectors or verified outputs and cannot be built here, so the
oracle is pinned by: an independent library (numpy.fft / numpy matmul), a brute-force O(D^2) DFT,
closed forms of the layer (impulse, constant, in-band / out-of-band tone) and invariants
(linearity, alpha scaling, channel-mix commutation, 2D separability). Each check is chosen so a
plausible slip (wrong sign, dropped alpha, transposed W, wrong mode window, wrong batch order)
fails at least one of them.
"""
import numpy as np
import pytest

import oracle
from conftest import rel_l2

RNG = np.random.default_rng(20240611)


def crand(*shape):
    return (RNG.uniform(-1, 1, shape) + 1j * RNG.uniform(-1, 1, shape)).astype(np.complex64)


def numpy_layer_1d(x, W, alpha):
    """independent evaluation with numpy.fft: x[K][S][DY], W[N][K]"""
    DY = x.shape[-1]
    A = np.fft.fft(x.astype(np.complex128), axis=-1)[..., :64]            # [K][S][64]
    C = alpha * np.einsum("ksm,nk->nsm", A, W.astype(np.complex128))
    Cp = np.zeros(C.shape[:-1] + (DY,), dtype=np.complex128)
    Cp[..., :64] = C
    return np.fft.ifft(Cp, axis=-1) * DY


def numpy_layer_2d(x, W, alpha):
    K, bs, DX, DY = x.shape
    A = np.fft.fft2(x.astype(np.complex128), axes=(-2, -1))[..., :64, :64]
    C = alpha * np.einsum("kbpq,nk->nbpq", A, W.astype(np.complex128))
    Cp = np.zeros((W.shape[0], bs, DX, DY), dtype=np.complex128)
    Cp[..., :64, :64] = C
    return np.fft.ifft2(Cp, axes=(-2, -1)) * (DX * DY)


@pytest.mark.parametrize("D", [2, 8, 64, 128, 256, 1024])
@pytest.mark.parametrize("sign", [-1, 1])
def test_fft_vs_numpy_and_bruteforce(D, sign):
    v = crand(3, D).astype(np.complex128)
    got = oracle.fft_batched(v, sign)
    ref = np.fft.fft(v, axis=-1) if sign < 0 else np.fft.ifft(v, axis=-1) * D
    assert rel_l2(got, ref) < 1e-13
    if D <= 256:
        brute = np.stack([oracle.dft_naive(v[i], sign) for i in range(3)])
        assert rel_l2(brute, ref) < 1e-12


def test_dft_naive_is_the_textbook_sum():
    # pins the brute-force routine itself, by hand, on D=4: forward of [1, i, -1, -i] is 4*delta[m-1]
    v = np.array([1, 1j, -1, -1j], dtype=np.complex128)
    np.testing.assert_allclose(oracle.dft_naive(v, -1), [0, 4, 0, 0], atol=1e-14)
    np.testing.assert_allclose(oracle.dft_naive(v, +1), [0, 0, 0, 4], atol=1e-14)


def test_cgemm_layout_and_alpha():
    K, N, M = 5, 3, 7
    A = crand(K, M).astype(np.complex128)
    W = crand(N, K).astype(np.complex128)
    alpha = 1.0 - 1.0j                       # the value the reference's drivers pass (fused.cu:76)
    got = oracle.cgemm(A, W, alpha)
    ref = alpha * (W @ A)                    # C[n][m] = sum_k W[n][k] A[k][m]
    assert rel_l2(got, ref) < 1e-14
    # a transposed W (W[n + k*N]) must NOT match
    wrong = alpha * (W.reshape(K, N).T @ A)
    assert rel_l2(got, wrong) > 1e-2


@pytest.mark.parametrize("DY", [128, 256, 512])
def test_trunc_and_pad_steps(DY):
    x = crand(6, DY)
    spec = oracle.fft_trunc_contig(x)
    assert spec.shape == (6, 64)
    assert rel_l2(spec, np.fft.fft(x.astype(np.complex128), axis=-1)[:, :64]) < 1e-13
    y = oracle.ifft_pad_contig(spec, DY)
    full = np.zeros((6, DY), dtype=np.complex128)
    full[:, :64] = spec
    assert rel_l2(y, np.fft.ifft(full, axis=-1) * DY) < 1e-13


@pytest.mark.parametrize("S,DY,K,N,alpha", [(1, 128, 8, 64, 1.0), (3, 256, 16, 64, 1 - 1j), (2, 128, 24, 128, 0.5j)])
def test_layer_1d_vs_numpy(S, DY, K, N, alpha):
    x = crand(K, S, DY)
    W = (crand(N, K) / np.sqrt(K)).astype(np.complex64)
    assert rel_l2(oracle.layer_1d(x, W, alpha), numpy_layer_1d(x, W, alpha)) < 1e-13


def test_layer_1d_closed_forms():
    K, S, DY, N = 8, 2, 128, 64
    W = (crand(N, K) / np.sqrt(K)).astype(np.complex64)
    Wd = W.astype(np.complex128)
    alpha = 1 - 1j
    # impulse at (k0, s0, j0):  y[n][s0][j] = alpha W[k0][n] D(j-j0),  D(d) = sum_{m<64} e^{2 pi i m d / DY}
    k0, s0, j0 = 3, 1, 17
    x = np.zeros((K, S, DY), dtype=np.complex64)
    x[k0, s0, j0] = 1
    y = oracle.layer_1d(x, W, alpha)
    d = np.arange(DY) - j0
    Dk = np.exp(2j * np.pi * np.outer(d, np.arange(64)) / DY).sum(axis=1)
    expect = np.zeros((N, S, DY), dtype=np.complex128)
    expect[:, s0, :] = alpha * Wd[:, k0][:, None] * Dk[None, :]
    assert rel_l2(y, expect) < 1e-12
    assert np.abs(y[:, 0, :]).max() < 1e-12            # other signal untouched
    # constant 1 in every channel: only bin 0 survives:  y = alpha * DY * sum_k W[k][n] for every j
    x = np.ones((K, S, DY), dtype=np.complex64)
    y = oracle.layer_1d(x, W, alpha)
    expect = np.broadcast_to((alpha * DY * Wd.sum(axis=1))[:, None, None], y.shape)
    assert rel_l2(y, expect) < 1e-12
    # pure tone at bin m: passes with gain DY for m < 64, is removed exactly for m >= 64
    j = np.arange(DY)
    for m, keep in [(5, True), (63, True), (64, False), (DY - 1, False)]:
        x = np.zeros((K, S, DY), dtype=np.complex128)
        x[2, 0, :] = np.exp(2j * np.pi * m * j / DY)
        x32 = x.astype(np.complex64)
        y = oracle.layer_1d(x32, W, alpha)
        if keep:
            expect = np.zeros_like(y)
            expect[:, 0, :] = alpha * DY * Wd[:, 2][:, None] * x32[2, 0, :].astype(np.complex128)[None, :]
            assert rel_l2(y, expect) < 1e-6        # fp32 rounding of the input tone
        else:
            assert np.abs(y).max() < 1e-4 * DY


def test_layer_1d_invariants():
    K, S, DY, N = 16, 2, 256, 64
    x1, x2 = crand(K, S, DY), crand(K, S, DY)
    W = (crand(N, K) / np.sqrt(K)).astype(np.complex64)
    y1, y2 = oracle.layer_1d(x1, W), oracle.layer_1d(x2, W)
    # exact-in-fp32 combination so linearity is not blurred by input rounding
    y12 = oracle.layer_1d((x1 + 2 * x2).astype(np.complex64), W)
    assert rel_l2(y12, y1 + 2 * y2) < 1e-6
    assert rel_l2(oracle.layer_1d(x1, W, 1 - 1j), (1 - 1j) * y1) < 1e-13
    # W is mode independent: layer == lowpass(sum_k W[k][n] x[k]) -- second evaluation order
    mix = np.einsum("ksj,nk->nsj", x1.astype(np.complex128), W.astype(np.complex128))
    spec = np.fft.fft(mix, axis=-1)
    spec[..., 64:] = 0
    assert rel_l2(y1, np.fft.ifft(spec, axis=-1) * DY) < 1e-12


@pytest.mark.parametrize("DX,DY", [(128, 128), (256, 128), (128, 256)])
def test_stride_steps_vs_numpy(DX, DY):
    x = crand(2, DX, DY)
    t1 = oracle.fft_stride(x)
    assert rel_l2(t1, np.fft.fft(x.astype(np.complex128), axis=1)[:, :64, :]) < 1e-13
    back = oracle.ifft_stride(t1, DX)
    full = np.zeros((2, DX, DY), dtype=np.complex128)
    full[:, :64, :] = t1
    assert rel_l2(back, np.fft.ifft(full, axis=1) * DX) < 1e-13


@pytest.mark.parametrize("bs,DX,DY,K,N,alpha", [(1, 128, 128, 8, 64, 1.0), (2, 128, 256, 16, 64, 1 - 1j)])
def test_layer_2d_vs_numpy(bs, DX, DY, K, N, alpha):
    x = crand(K, bs, DX, DY)
    W = (crand(N, K) / np.sqrt(K)).astype(np.complex64)
    assert rel_l2(oracle.layer_2d(x, W, alpha), numpy_layer_2d(x, W, alpha)) < 1e-13


def test_layer_2d_closed_forms_and_separability():
    K, bs, DX, DY, N = 8, 1, 128, 128, 64
    W = (crand(N, K) / np.sqrt(K)).astype(np.complex64)
    Wd = W.astype(np.complex128)
    # impulse at (k0,b,x0,y0): y = alpha W[k0][n] Dx(x-x0) Dy(y-y0)  (separable Dirichlet kernels)
    x = np.zeros((K, bs, DX, DY), dtype=np.complex64)
    x[1, 0, 9, 40] = 1
    y = oracle.layer_2d(x, W, 1.0)
    Dx = np.exp(2j * np.pi * np.outer(np.arange(DX) - 9, np.arange(64)) / DX).sum(axis=1)
    Dy = np.exp(2j * np.pi * np.outer(np.arange(DY) - 40, np.arange(64)) / DY).sum(axis=1)
    expect = Wd[:, 1][:, None, None, None] * (Dx[:, None] * Dy[None, :])[None, None]
    assert rel_l2(y, expect) < 1e-12
    # tone in band along X but out of band along Y must vanish (mode window is p<64 AND q<64)
    xx, yy = np.meshgrid(np.arange(DX), np.arange(DY), indexing="ij")
    x = np.zeros((K, bs, DX, DY), dtype=np.complex64)
    x[0, 0] = np.exp(2j * np.pi * (3 * xx / DX + 70 * yy / DY)).astype(np.complex64)
    assert np.abs(oracle.layer_2d(x, W, 1.0)).max() < 1e-3
    x[0, 0] = np.exp(2j * np.pi * (3 * xx / DX + 7 * yy / DY)).astype(np.complex64)
    y = oracle.layer_2d(x, W, 1.0)
    expect = DX * DY * Wd[:, 0][:, None, None, None] * x[0, 0].astype(np.complex128)[None, None]
    assert rel_l2(y, expect) < 1e-6


def test_cpu_baseline_matches_oracle():
    # the fp32 OpenMP baseline (timed by the benchmark) computes the same layer
    x = crand(8, 2, 128)
    W = (crand(64, 8) / np.sqrt(8)).astype(np.complex64)
    assert rel_l2(oracle.cpu_baseline_layer_1d(x, W, 1 - 1j, 2), oracle.layer_1d(x, W, 1 - 1j)) < 1e-5
    x = crand(8, 1, 128, 128)
    assert rel_l2(oracle.cpu_baseline_layer_2d(x, W, 1.0, 2), oracle.layer_2d(x, W, 1.0)) < 1e-5
