"""GPU checks at the full sizes of the benchmark configurations.

Where the CPU oracle finishes in seconds (all 1D configurations) the HIP path is compared with it directly; at the
2D sizes it is compared with an independent library evaluation on the GPU (rocFFT through torch.fft plus a torch
contraction, complex64) and through properties that do not depend on size: linearity in x, agreement of the two
independent 2D algorithms, and idempotence of the layer when it is a pure low-pass projection.
"""
import numpy as np
import pytest
import torch

import oracle
import turbofno_amd as tf
from turbofno_amd import workloads
from conftest import max_rel, rel_l2

pytestmark = pytest.mark.gpu


def _rel(a, b):
    return float(torch.linalg.vector_norm(a - b) / torch.linalg.vector_norm(b))


def _library_layer_2d(x, W, alpha=1.0):
    K, bs, DX, DY = x.shape
    N = W.shape[0]
    A = torch.fft.fft2(x)[..., :64, :64]
    C = alpha * torch.einsum("kbpq,nk->nbpq", A, W)
    Cp = torch.zeros((N, bs, DX, DY), dtype=torch.complex64, device=x.device)
    Cp[..., :64, :64] = C
    return torch.fft.ifft2(Cp, norm="forward")


def test_config2_sweep_against_oracle(tol):
    """the whole 1D grid of configuration 2: bs x DY x N x K = 7 x 2 x 2 x 4 = 112 problems"""
    worst = 0.0
    for bs in (1, 2, 4, 8, 16, 32, 64):
        for DY in (128, 256):
            for N in (64, 128):
                for K in (8, 16, 24, 32):
                    print("config2", bs, DY, N, K, flush=True)
                    x, W = workloads.uniform_1d(1000 + bs + DY + N + K, bs, DY, K, N)
                    y = tf.layer_1d(torch.from_numpy(x).cuda(), torch.from_numpy(W).cuda()).cpu().numpy()
                    ref = oracle.layer_1d(x, W, 1.0)
                    e2, em = rel_l2(y, ref), max_rel(y, ref)
                    worst = max(worst, e2)
                    assert e2 <= tol["l2"] and em <= tol["max"], (bs, DY, N, K, e2, em)
    print("worst rel_l2 %.3e" % worst)


@pytest.mark.parametrize("K", [64, 128])
@pytest.mark.parametrize("algo", [0, 1, 2, 3, 4, 5, 6])
def test_config3_large_hidden_against_oracle(K, algo, tol, monkeypatch):
    """1D bs=64, DY=256, N=128, K in {64, 128}, smooth input: size-chosen kernel, SIMT kernel, the three matrix-core variants"""
    print("config3", K, algo, flush=True)
    monkeypatch.setenv("TURBOFNO_1D_ALGO", str(algo))
    x, W = workloads.smooth_1d(0x5EED + 3, 64, 256, K, 128)
    y = tf.layer_1d(torch.from_numpy(x).cuda(), torch.from_numpy(W).cuda()).cpu().numpy()
    ref = oracle.layer_1d(x, W, 1.0)
    assert rel_l2(y, ref) <= tol["l2"] and max_rel(y, ref) <= tol["max"]


@pytest.mark.parametrize("bs", [1, 4, 16])
@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("K", [16, 32])
def test_config4_grid_against_library(bs, D, K, tol):
    print("config4", bs, D, K, flush=True)
    x_h, W_h = workloads.uniform_2d(400 + bs + D + K, bs, D, D, K, 64)
    x, W = torch.from_numpy(x_h).cuda(), torch.from_numpy(W_h).cuda()
    ref = _library_layer_2d(x, W)
    for algo in (0, 1, 2):
        y = tf.layer_2d(x, W, algo=algo)
        torch.cuda.synchronize()
        assert _rel(y, ref) <= tol["l2"], (algo, _rel(y, ref))
        assert float((y - ref).abs().max() / ref.abs().max()) <= tol["max"]


@pytest.fixture(scope="module")
def headline():
    x_h, W_h = workloads.vorticity_2d(0x5EED + 5, 16, 256, 256, 64, 64)
    return torch.from_numpy(x_h).cuda(), torch.from_numpy(W_h).cuda()


def test_headline_against_library(headline, tol):
    x, W = headline
    print("headline vs rocFFT + torch contraction", flush=True)
    ref = _library_layer_2d(x, W)
    y = tf.layer_2d(x, W)
    torch.cuda.synchronize()
    assert _rel(y, ref) <= tol["l2"], _rel(y, ref)
    assert float((y - ref).abs().max() / ref.abs().max()) <= tol["max"]


def test_headline_two_algorithms_agree(headline, tol):
    x, W = headline
    print("headline whole-image vs three-kernel", flush=True)
    y2 = tf.layer_2d(x, W, algo=2)
    y1 = tf.layer_2d(x, W, algo=1)
    torch.cuda.synchronize()
    assert _rel(y2, y1) <= tol["l2"], _rel(y2, y1)


def test_headline_linearity(headline, tol):
    x, W = headline
    print("headline linearity", flush=True)
    x2 = torch.roll(x, shifts=(3, 17), dims=(2, 3)).contiguous()
    a, b = 0.75 - 0.5j, -1.25 + 0.25j
    lhs = tf.layer_2d((a * x + b * x2).contiguous(), W)
    rhs = a * tf.layer_2d(x, W) + b * tf.layer_2d(x2, W)
    torch.cuda.synchronize()
    assert _rel(lhs, rhs) <= 2 * tol["l2"], _rel(lhs, rhs)


def test_headline_lowpass_is_idempotent(headline, tol):
    """W = identity, alpha = 1/(DX DY): the layer is the projection onto the 64 x 64 lowest modes, so applying it
    twice changes nothing, and it removes exactly the energy of the discarded modes (Parseval)."""
    x, _ = headline
    print("headline idempotence", flush=True)
    W = torch.eye(64, dtype=torch.complex64, device="cuda")
    alpha = 1.0 / (256 * 256)
    y1 = tf.layer_2d(x, W, alpha=alpha)
    y2 = tf.layer_2d(y1, W, alpha=alpha)
    torch.cuda.synchronize()
    assert _rel(y2, y1) <= 2 * tol["l2"], _rel(y2, y1)
    spec = torch.fft.fft2(x[:4])
    kept = torch.linalg.vector_norm(spec[..., :64, :64]) ** 2 / (256 * 256)
    assert abs(float(torch.linalg.vector_norm(y1[:4]) ** 2 / kept) - 1.0) <= 1e-4
