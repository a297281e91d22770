"""Out-of-bounds writes: every output (and the 2D workspace) sits between two guard bands filled with a canary; after
the call the bands must be untouched. Shapes are chosen so that the last block / chunk / image pass is partial."""
import numpy as np
import pytest
import torch

import turbofno_amd as tf
from turbofno_amd import workloads

pytestmark = pytest.mark.gpu
PAD = 4096                      # complex elements on either side
CANARY = complex(-7.25, 3.5)


def guarded(shape):
    n = int(np.prod(shape))
    buf = torch.full((n + 2 * PAD,), CANARY, dtype=torch.complex64, device="cuda")
    return buf, buf[PAD:PAD + n].view(shape)


def intact(buf, what):
    torch.cuda.synchronize()
    lo, hi = buf[:PAD], buf[-PAD:]
    assert bool((lo == CANARY).all()) and bool((hi == CANARY).all()), what + ": guard band overwritten"


@pytest.mark.parametrize("algo", [0, 1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("bs,DY,K,N", [(3, 256, 72, 128), (5, 128, 40, 64), (1, 256, 8, 64), (7, 128, 136, 128),
                                       (5, 256, 64, 128), (13, 256, 192, 64)])
def test_layer_1d_stays_in_bounds(bs, DY, K, N, algo, algo_1d):
    print("guard 1d", bs, DY, K, N, algo, flush=True)
    algo_1d(algo)
    x_h, W_h = workloads.uniform_1d(70 + bs + K, bs, DY, K, N)
    buf, y = guarded((N, bs, DY))
    tf.layer_1d(torch.from_numpy(x_h).cuda(), torch.from_numpy(W_h).cuda(), y=y)
    intact(buf, "layer_1d")
    assert not bool((y == CANARY).any())            # and the output itself was written everywhere


@pytest.mark.parametrize("algo", [1, 2, 3])
@pytest.mark.parametrize("bs,DX,DY,K,N", [(3, 128, 256, 24, 64), (1, 256, 128, 72, 128), (5, 128, 128, 8, 64),
                                          (2, 256, 256, 40, 64)])
def test_layer_2d_stays_in_bounds(bs, DX, DY, K, N, algo):
    print("guard 2d", bs, DX, DY, K, N, algo, flush=True)
    x_h, W_h = workloads.uniform_2d(80 + bs + K, bs, DX, DY, K, N)
    buf, y = guarded((N, bs, DX, DY))
    need = tf.layer_2d_workspace_bytes(bs, DX, DY, K, N, algo)
    wbuf = torch.full((need // 8 + 2 * PAD,), CANARY, dtype=torch.complex64, device="cuda")
    ws = wbuf[PAD:PAD + need // 8].view(torch.uint8)
    tf.layer_2d(torch.from_numpy(x_h).cuda(), torch.from_numpy(W_h).cuda(), y=y, workspace=ws, algo=algo)
    intact(buf, "layer_2d output")
    intact(wbuf, "layer_2d workspace")
    assert not bool((y == CANARY).any())


@pytest.mark.parametrize("M,N,K", [(64, 64, 8), (192, 128, 72), (4160, 64, 16), (1024, 64, 48), (320, 64, 128)])
def test_cgemm_stays_in_bounds(M, N, K):
    print("guard cgemm", M, N, K, flush=True)
    rng = np.random.default_rng(M + K)
    A = torch.from_numpy((rng.uniform(-1, 1, (K, M)) + 1j * rng.uniform(-1, 1, (K, M))).astype(np.complex64)).cuda()
    W = torch.from_numpy((rng.uniform(-1, 1, (N, K)) + 1j * rng.uniform(-1, 1, (N, K))).astype(np.complex64)).cuda()
    buf, C = guarded((N, M))
    tf.cgemm(M, N, K, A, W, C, 1.0, 0.0)
    intact(buf, "cgemm")
    ref = torch.einsum("nk,km->nm", W, A)
    assert float(torch.linalg.vector_norm(C - ref) / torch.linalg.vector_norm(ref)) <= 1e-5


@pytest.mark.parametrize("D,other,nsig", [(128, 48, 3), (256, 16, 5), (512, 32, 2), (1024, 16, 1), (256, 96, 3), (128, 64, 2)])
def test_stride_kernels_stay_in_bounds(D, other, nsig):
    print("guard stride", D, other, nsig, flush=True)
    rng = np.random.default_rng(D)
    x = torch.from_numpy((rng.uniform(-1, 1, (nsig, D, other)) + 0j).astype(np.complex64)).cuda()
    b1, t1 = guarded((nsig, 64, other))
    tf.fft_stride(x, t1, 4, other, other * nsig, 64)
    intact(b1, "fft_stride")
    b2, back = guarded((nsig, D, other))
    tf.ifft_stride(t1.contiguous(), back, 4, other, other * nsig, 64)
    intact(b2, "ifft_stride")
    xs = torch.from_numpy((rng.uniform(-1, 1, (nsig * 3, D)) + 0j).astype(np.complex64)).cuda()
    b3, a = guarded((nsig * 3, 64))
    tf.fft_stride_DY(xs, a, 4, nsig * 3)
    intact(b3, "fft_stride_DY")
    b4, yy = guarded((nsig * 3, D))
    tf.ifft_stride_DY(a.contiguous(), yy, 4, nsig * 3)
    intact(b4, "ifft_stride_DY")
