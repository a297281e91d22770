"""GPU checks at the full sizes of the benchmark configurations.

Where the CPU oracle finishes in seconds (all 1D configurations) the HIP path is compared with it directly. At the
2D sizes batch elements are independent, so the full-size run on the GPU is compared with the oracle on slices:
y[:, b] against oracle.layer_2d(x[:, b:b+1], W) for a few b. In addition it is compared with an independent library
evaluation on the GPU (rocFFT through torch.fft plus a torch contraction, complex64) and through properties that do
not depend on size: linearity in x, agreement of the two independent 2D algorithms, and idempotence of the layer when
it is a pure low-pass projection.
"""
import numpy as np
import pytest
import torch

import oracle
import turbofno_amd as tf
from turbofno_amd import workloads
from conftest import max_rel, max_rel_elementwise, rel_l2

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
@pytest.mark.parametrize("algo", [0, 1, 2, 3, 4, 5, 6, 7, 8])
def test_config3_large_hidden_against_oracle(K, algo, tol, algo_1d):
    """1D bs=64, DY=256, N=128, K in {64, 128}, smooth input: size-chosen kernel, SIMT kernel, the three matrix-core variants"""
    print("config3", K, algo, flush=True)
    algo_1d(algo)
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


def _check_batch_slices(y, x_h, W_h, alpha, batch_elements, tol, what):
    """y[:, b] of a full-size GPU result against the fp64 oracle run on batch element b alone"""
    for b in batch_elements:
        ref = oracle.layer_2d(np.ascontiguousarray(x_h[:, b:b + 1]), W_h, alpha)
        got = y[:, b:b + 1].cpu().numpy()
        e2, em, ee = rel_l2(got, ref), max_rel(got, ref), max_rel_elementwise(got, ref)
        print("%s b=%d rel_l2=%.3e max_rel=%.3e elementwise=%.3e" % (what, b, e2, em, ee), flush=True)
        assert e2 <= tol["l2"] and em <= tol["max"] and ee <= tol["elem"], (what, b, e2, em, ee)


@pytest.mark.parametrize("algo", [0, 1, 2, 3])
def test_headline_against_oracle_slices(algo, tol):
    """configuration 5 (bs=16, 256 x 256, K=N=64, Gaussian random field) at full size; batch elements 0, 7, 15
    against the oracle"""
    print("headline vs oracle slices, algo", algo, flush=True)
    x_h, W_h = workloads.vorticity_2d(0x5EED + 5, 16, 256, 256, 64, 64)
    y = tf.layer_2d(torch.from_numpy(x_h).cuda(), torch.from_numpy(W_h).cuda(), algo=algo)
    torch.cuda.synchronize()
    _check_batch_slices(y, x_h, W_h, 1.0, (0, 7, 15), tol, "headline algo %d" % algo)


@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("K", [16, 32])
def test_config4_bs16_against_oracle_slices(D, K, tol):
    """configuration 4 at its largest batch, every algorithm, batch elements 0, 5, 15 against the oracle"""
    x_h, W_h = workloads.uniform_2d(440 + D + K, 16, D, D, K, 64)
    x, W = torch.from_numpy(x_h).cuda(), torch.from_numpy(W_h).cuda()
    for algo in (0, 1, 2, 3):
        print("config4 bs=16 vs oracle slices", D, K, "algo", algo, flush=True)
        y = tf.layer_2d(x, W, alpha=1 - 1j, algo=algo)
        torch.cuda.synchronize()
        _check_batch_slices(y, x_h, W_h, 1 - 1j, (0, 5, 15), tol, "config4 D=%d K=%d algo %d" % (D, K, algo))


@pytest.mark.parametrize("bs", [1, 4])
@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("K", [16, 32])
def test_config4_small_batches_against_oracle(bs, D, K, tol):
    """configuration 4 at bs = 1 and 4: the algorithm chosen by size (three kernels) and the other two, every batch
    element against the oracle; the choice itself is asserted, so that a change of the rule shows up here"""
    assert tf.query_2d_algo(bs, D, D, K, 64) == tf.ALGO_THREE_KERNEL
    x_h, W_h = workloads.uniform_2d(470 + bs + D + K, bs, D, D, K, 64)
    x, W = torch.from_numpy(x_h).cuda(), torch.from_numpy(W_h).cuda()
    for algo in (0, 2, 3):
        print("config4 small batch vs oracle", bs, D, K, "algo", algo, flush=True)
        y = tf.layer_2d(x, W, alpha=0.5 + 1j, algo=algo)
        torch.cuda.synchronize()
        _check_batch_slices(y, x_h, W_h, 0.5 + 1j, range(bs), tol, "config4 bs=%d D=%d K=%d algo %d" % (bs, D, K, algo))


@pytest.mark.parametrize("bs,DX,DY,K,N,algo", [
    (4, 512, 512, 32, 64, 0),        # 768 MiB of 512 x 512: the whole-image kernels by size (768 + 1024 parts of 256 x 512)
    (4, 512, 512, 32, 64, 3),        # whole rows first: 2048 row blocks of 32 rows on at most 768 persistent blocks
    (4, 256, 1024, 32, 64, 0),       # DY > DX: whole rows first, eight batches of rows per block
    (4, 1024, 256, 32, 64, 0),       # DX > DY: X axis first
    (6, 512, 512, 24, 128, 1),
    (6, 512, 512, 24, 128, 3),
    (6, 512, 256, 24, 128, 2),       # whole-image kernels, several parts per persistent block: two parts per image, ...
    (3, 1024, 512, 24, 64, 2),       # ... four parts and rows of 512, ...
    (5, 256, 1024, 40, 128, 2),      # ... rows of 1024
])
def test_large_images_against_oracle_slices(bs, DX, DY, K, N, algo, tol):
    """lengths above 256 at sizes that run the persistent loops of the X-axis kernels, of the row kernels and of the
    whole-image kernels several times per block; first and last batch element against the oracle"""
    print("large images", bs, DX, DY, K, N, "algo", algo, flush=True)
    x_h, W_h = workloads.uniform_2d(950 + bs + DX + K + algo, bs, DX, DY, K, N)
    y = tf.layer_2d(torch.from_numpy(x_h).cuda(), torch.from_numpy(W_h).cuda(), alpha=0.5 - 1j, algo=algo)
    torch.cuda.synchronize()
    _check_batch_slices(y, x_h, W_h, 0.5 - 1j, (0, bs - 1), tol, "large images %dx%d algo %d" % (DX, DY, algo))


@pytest.mark.parametrize("bs,DX,DY,K,N", [
    (5, 256, 256, 64, 64),           # 320 input images on a 256-block persistent grid: 64 blocks take a second image
    (9, 256, 256, 64, 128),          # 576 input and 1152 output images: up to three / five images per block
    (11, 128, 256, 56, 64),          # 616 images of 128 x 256, K not a multiple of 16
    (10, 256, 128, 64, 64),          # 640 images with paired rows of 128
])
def test_whole_image_persistent_loop_against_oracle(bs, DX, DY, K, N, tol):
    """more images than persistent blocks, so that the image loop of the whole-image kernels and its look-ahead
    loads across the image boundary run several times per block; a spread of batch elements against the oracle"""
    print("whole-image persistent loop", bs, DX, DY, K, N, flush=True)
    x_h, W_h = workloads.uniform_2d(900 + bs + DX + K, bs, DX, DY, K, N)
    y = tf.layer_2d(torch.from_numpy(x_h).cuda(), torch.from_numpy(W_h).cuda(), alpha=0.5 + 0.25j, algo=2)
    torch.cuda.synchronize()
    _check_batch_slices(y, x_h, W_h, 0.5 + 0.25j, sorted({0, 1, bs // 2, bs - 2, bs - 1}), tol, "persistent loop")


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
