"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs.

Tolerances are the ones the build's baseline states for complex fp32: relative L2 <= 1e-5 and max
element error <= 1e-4 (relative to the largest reference magnitude).
"""
import numpy as np
import pytest
import torch

import oracle
import turbofno_amd as tf
from turbofno_amd import workloads
from conftest import max_rel, max_rel_elementwise, rel_l2

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def check(got, ref, tol, what=""):
    got = got.cpu().numpy()
    e2, em, ee = rel_l2(got, ref), max_rel(got, ref), max_rel_elementwise(got, ref)
    print("%s rel_l2=%.3e max_rel=%.3e elementwise=%.3e" % (what, e2, em, ee), flush=True)
    assert e2 <= tol["l2"], (what, e2)
    assert em <= tol["max"], (what, em)
    assert ee <= tol["elem"], (what, ee)


@pytest.mark.parametrize("bs,DY,K,N,alpha", [
    (1, 128, 8, 64, 1.0),            # config 1 (plumbing case); K=8 < chunk -> zero-filled tail
    (1, 256, 8, 64, 1 - 1j),         # alpha the reference's drivers pass (fused.cu:76)
    (3, 128, 24, 128, 1.0),          # K not a multiple of the 32-channel chunk, two N tiles
    (5, 256, 24, 64, 1.0),           # K not a multiple of the 16-channel chunk
    (16, 256, 32, 128, 0.5j),
    (64, 128, 16, 64, 1.0),
    (3, 512, 24, 64, 1 - 1j),        # lengths 512 / 1024: 32 / 64 lanes per signal, chunks of 8 / 4 channels
    (2, 1024, 8, 128, 1.0),
    (5, 1024, 40, 64, 0.5j),
])
def test_layer_1d(bs, DY, K, N, alpha, tol):
    print("case layer_1d", bs, DY, K, N, alpha, flush=True)
    x, W = workloads.uniform_1d(7 + bs + DY + K, bs, DY, K, N)
    y = tf.layer_1d(dev(x), dev(W), alpha=alpha)
    torch.cuda.synchronize()
    check(y, oracle.layer_1d(x, W, alpha), tol, "layer_1d")


@pytest.mark.parametrize("algo", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("bs,DY,K,N,alpha", [
    (2, 256, 32, 64, 1.0),           # exactly one chunk of the matrix-core kernel
    (3, 256, 72, 128, 1 - 1j),       # chunks 32 + 32 + 8, two N tiles
    (2, 256, 8, 64, 1.0),            # K smaller than a chunk
    (4, 128, 64, 64, 1.0),           # DY=128: one chunk of 64 channels
    (3, 128, 72, 128, 0.5j),         # DY=128: 64 + 8
    (2, 256, 128, 128, 1.0),         # large-hidden shape
])
def test_layer_1d_both_contractions(bs, DY, K, N, alpha, algo, tol, algo_1d):
    """the SIMT and the matrix-core fused kernels, forced through turbofno_set_1d_algo, on the same problems"""
    print("case layer_1d algo", algo, bs, DY, K, N, alpha, flush=True)
    algo_1d(algo)
    x, W = workloads.smooth_1d(11 + bs + DY + K, bs, DY, K, N)
    y = tf.layer_1d(dev(x), dev(W), alpha=alpha)
    torch.cuda.synchronize()
    check(y, oracle.layer_1d(x, W, alpha), tol, "layer_1d algo %d" % algo)


@pytest.mark.parametrize("seed", range(36))
def test_layer_1d_random_shapes(seed, tol, algo_1d):
    """seeded random shapes (odd S, three N tiles, K up to 136, complex alpha) through every 1D kernel choice"""
    rng = np.random.default_rng(1000 + seed)
    DY = int(rng.choice([128, 256]))
    K = 8 * int(rng.integers(1, 18))
    N = 64 * int(rng.integers(1, 4))
    S = int(rng.integers(1, 41))
    algo = seed % 9
    alpha = complex(rng.uniform(-1, 1), rng.uniform(-1, 1))
    print("case layer_1d random", seed, "S", S, "DY", DY, "K", K, "N", N, "algo", algo, flush=True)
    algo_1d(algo)
    x, W = workloads.uniform_1d(seed, S, DY, K, N)
    y = tf.layer_1d(dev(x), dev(W), alpha=alpha)
    torch.cuda.synchronize()
    check(y, oracle.layer_1d(x, W, alpha), tol, "layer_1d random %d" % seed)


@pytest.mark.parametrize("bs,DY,K,N", [
    (1030, 128, 16, 64),             # DY=128: from two items per CU on for K <= 16
    (600, 128, 40, 128),             # DY=128, 1200 items, K = 5 rounds of 8 channels
    (2100, 256, 8, 64),              # DY=256: from eight items per CU on
    (1040, 256, 72, 128),            # DY=256, 2080 items, two N tiles, K = 18 rounds of 4 channels
])
def test_layer_1d_large_grids(bs, DY, K, N, tol):
    """grids large enough for the size rule to pick the one-wavefront-per-item kernel (on a 256-CU device)"""
    print("case layer_1d large grid", bs, DY, K, N, flush=True)
    x, W = workloads.uniform_1d(3 + bs + DY + K, bs, DY, K, N)
    y = tf.layer_1d(dev(x), dev(W), alpha=1 - 1j)
    torch.cuda.synchronize()
    check(y, oracle.layer_1d(x, W, 1 - 1j), tol, "layer_1d large grid")


@pytest.mark.parametrize("DX,DY,nsig", [(128, 128, 3), (256, 128, 2), (128, 256, 2), (256, 256, 2),
                                        (512, 32, 3), (1024, 48, 2)])
def test_stride_stages(DX, DY, nsig, tol):
    print("case stride", DX, DY, nsig, flush=True)
    rng = np.random.default_rng(DX + DY)
    x = (rng.uniform(-1, 1, (nsig, DX, DY)) + 1j * rng.uniform(-1, 1, (nsig, DX, DY))).astype(np.complex64)
    t1 = torch.empty((nsig, 64, DY), dtype=torch.complex64, device="cuda")
    tf.fft_stride(dev(x), t1, 4, DY, DY * nsig, 64)
    torch.cuda.synchronize()
    ref_t1 = oracle.fft_stride(x)
    check(t1, ref_t1, tol, "fft_stride")
    back = torch.empty((nsig, DX, DY), dtype=torch.complex64, device="cuda")
    t1_in = ref_t1.astype(np.complex64)
    tf.ifft_stride(dev(t1_in), back, 4, DY, DY * nsig, 64)
    torch.cuda.synchronize()
    check(back, oracle.ifft_stride(t1_in.astype(np.complex128), DX), tol, "ifft_stride")


@pytest.mark.parametrize("bs,DX,DY,K,N,algo", [
    (1, 128, 128, 16, 64, 1),
    (2, 256, 128, 8, 64, 1),
    (1, 128, 256, 16, 64, 1),
    (1, 256, 256, 16, 64, 1),
    (1, 256, 256, 16, 64, 2),
    (2, 256, 256, 8, 128, 2),
    (1, 256, 256, 72, 64, 2),        # K above 64: GEMM in chunks of 32 channels (32 + 32 + 8)
    (1, 128, 128, 128, 64, 2),       # four full chunks
    (1, 128, 128, 104, 128, 2),      # 32 + 32 + 32 + 8, two N tiles
    (1, 128, 128, 40, 64, 2),        # one chunk, 12 channel groups (last one half empty)
    (1, 128, 128, 64, 64, 2),        # one full chunk
    (1, 128, 128, 16, 64, 2),        # whole-image kernels for the other three built shapes
    (3, 128, 256, 8, 64, 2),
    (2, 256, 128, 24, 128, 2),
    (5, 128, 128, 8, 64, 0),         # auto: 40 input images, below the whole-image threshold -> three-kernel path
    (1, 512, 128, 8, 64, 0),         # lengths above 256, DX > DY: auto = three-kernel path (X axis first)
    (1, 256, 1024, 16, 64, 1),
    (2, 1024, 512, 8, 64, 0),
    (1, 256, 1024, 16, 64, 0),       # DY > DX: auto = whole rows first
    (1, 512, 512, 8, 64, 0),         # square, few images: X axis first
    (2, 512, 512, 64, 64, 0),        # square, K * bs = 128: whole rows first
    (1, 1024, 1024, 8, 64, 0),
    (1, 128, 128, 16, 64, 3),        # whole rows first on every pair of lengths (row blocks of 32 rows, one to eight batches)
    (2, 256, 128, 8, 64, 3),
    (3, 128, 256, 24, 128, 3),
    (1, 256, 256, 72, 64, 3),
    (1, 512, 256, 8, 64, 3),
    (2, 128, 512, 16, 64, 3),
    (1, 1024, 128, 8, 64, 3),
    (1, 512, 1024, 8, 128, 3),
    (5, 128, 128, 8, 64, 3),         # 20 row blocks of 32 rows over 40 images: several images per persistent block
    (1, 512, 128, 8, 64, 2),         # whole-image path with DX above 256: two / four decimated parts of 256 rows per image,
    (2, 512, 256, 16, 64, 2),        # summed over by the contraction (2 K or 4 K channels: one chunk, ...
    (1, 1024, 256, 8, 64, 2),
    (1, 1024, 128, 24, 128, 2),      # ... 96 channels in chunks of 32, ...
    (3, 512, 256, 40, 64, 2),        # ... 80 = 32 + 32 + 16, ...
    (1, 1024, 256, 72, 64, 2),       # ... 288 channels: nine chunks)
    (1, 128, 512, 8, 64, 2),         # whole-image path with rows of 512 / 1024: 32 / 64 lanes per row
    (1, 256, 512, 16, 64, 2),
    (2, 128, 1024, 8, 64, 2),
    (1, 256, 1024, 24, 128, 2),
    (1, 512, 512, 8, 64, 2),         # both: long rows and interleaved parts
    (1, 1024, 512, 8, 64, 2),
    (1, 512, 1024, 40, 64, 2),
    (1, 1024, 1024, 8, 64, 2),
])
def test_layer_2d(bs, DX, DY, K, N, algo, tol):
    print("case layer_2d", bs, DX, DY, K, N, algo, flush=True)
    x, W = workloads.uniform_2d(11 + DX + DY + K + N, bs, DX, DY, K, N)
    alpha = 1 - 1j if K == 8 else 1.0
    y = tf.layer_2d(dev(x), dev(W), alpha=alpha, algo=algo)
    torch.cuda.synchronize()
    check(y, oracle.layer_2d(x, W, alpha), tol, "layer_2d algo=%d" % algo)


@pytest.mark.parametrize("seed", range(16))
def test_layer_2d_random_shapes(seed, tol):
    """seeded random 2D shapes through the size rule, the three-kernel path, the whole-image path and whole rows first"""
    rng = np.random.default_rng(2000 + seed)
    DX, DY = int(rng.choice([128, 256])), int(rng.choice([128, 256]))
    K = 8 * int(rng.integers(1, 12))
    N = 64 * int(rng.integers(1, 3))
    bs = int(rng.integers(1, 4))
    algo = seed % 4
    alpha = complex(rng.uniform(-1, 1), rng.uniform(-1, 1))
    print("case layer_2d random", seed, "bs", bs, DX, DY, "K", K, "N", N, "algo", algo, flush=True)
    x, W = workloads.uniform_2d(seed, bs, DX, DY, K, N)
    y = tf.layer_2d(dev(x), dev(W), alpha=alpha, algo=algo)
    torch.cuda.synchronize()
    check(y, oracle.layer_2d(x, W, alpha), tol, "layer_2d random %d" % seed)


@pytest.mark.parametrize("seed", range(12))
def test_layer_2d_random_long_shapes(seed, tol):
    """seeded random 2D shapes with at least one axis of 512 or 1024, through every algorithm: the three-stage paths and
    the whole-image kernels with their interleaved parts (DX above 256) and their 32- / 64-lane rows (DY above 256);
    first batch element against the oracle"""
    rng = np.random.default_rng(3000 + seed)
    lengths = [128, 256, 512, 1024]
    while True:
        DX, DY = int(rng.choice(lengths)), int(rng.choice(lengths))
        if max(DX, DY) > 256 and DX * DY <= 512 * 1024:
            break
    K = 8 * int(rng.integers(1, 6))
    N = 64 * int(rng.integers(1, 3))
    bs = int(rng.integers(1, 4))
    algo = (2, 2, 1, 3, 0, 2)[seed % 6]
    alpha = complex(rng.uniform(-1, 1), rng.uniform(-1, 1))
    print("case layer_2d random long", seed, "bs", bs, DX, DY, "K", K, "N", N, "algo", algo, flush=True)
    x, W = workloads.uniform_2d(seed, bs, DX, DY, K, N)
    y = tf.layer_2d(dev(x), dev(W), alpha=alpha, algo=algo)
    torch.cuda.synchronize()
    check(y[:, :1], oracle.layer_2d(np.ascontiguousarray(x[:, :1]), W, alpha), tol, "layer_2d random long %d" % seed)


def test_layer_2d_closed_forms(tol):
    """impulse and in-band tone through the whole-image path (analytic expectations, no oracle)."""
    K, bs, D, N = 8, 1, 256, 64
    rng = np.random.default_rng(5)
    W = workloads.weights_uniform(rng, N, K)
    x = np.zeros((K, bs, D, D), dtype=np.complex64)
    x[3, 0, 9, 200] = 1
    y = tf.layer_2d(dev(x), dev(W), algo=2).cpu().numpy()
    Dx = np.exp(2j * np.pi * np.outer(np.arange(D) - 9, np.arange(64)) / D).sum(axis=1)
    Dy = np.exp(2j * np.pi * np.outer(np.arange(D) - 200, np.arange(64)) / D).sum(axis=1)
    expect = W.astype(np.complex128)[:, 3][:, None, None, None] * (Dx[:, None] * Dy[None, :])[None, None]
    assert rel_l2(y, expect) <= tol["l2"]


def test_error_codes():
    x = torch.zeros((8, 1, 128), dtype=torch.complex64, device="cuda")
    W = torch.zeros((64, 8), dtype=torch.complex64, device="cuda")
    with pytest.raises(tf.TurboFNOError) as e:
        tf.layer_1d(x[:4].contiguous(), W[:, :4].contiguous())     # K = 4
    assert e.value.code == 1
    with pytest.raises(tf.TurboFNOError) as e:
        tf.layer_1d(torch.zeros((8, 1, 2048), dtype=torch.complex64, device="cuda"), W)
    assert e.value.code == 2
    x2 = torch.zeros((8, 1, 2048, 128), dtype=torch.complex64, device="cuda")
    with pytest.raises(tf.TurboFNOError) as e:                     # no 2D kernel of that length, whatever the algorithm
        tf.layer_2d(x2, W, algo=2)
    assert e.value.code == 2


@pytest.mark.parametrize("S,DY,K,N", [(4, 128, 8, 64), (8, 256, 24, 128), (1, 128, 16, 64), (5, 256, 8, 64),
                                      (3, 512, 16, 64), (2, 1024, 8, 64), (5, 128, 64, 64), (3, 128, 104, 128)])
def test_unfused_and_half_fused_stages(S, DY, K, N, tol):
    """stages of variants A, B, C: contiguous transforms, cgemm with beta, the two half-fused kernels"""
    print("case variant stages", S, DY, K, N, flush=True)
    x, W = workloads.uniform_1d(S + DY + K, S, DY, K, N)
    M = 64 * S
    alpha, beta = 1 - 1j, -1 + 1j                       # the values the reference's drivers pass
    # A = FFT_trunc(x): [K*S][DY] -> [K*S][64]  (= column-major M x K matrix)
    A = torch.empty((K, S, 64), dtype=torch.complex64, device="cuda")
    tf.fft_stride_DY(dev(x), A, 4, K * S)
    torch.cuda.synchronize()
    A_ref = oracle.fft_trunc_contig(x)
    check(A, A_ref, tol, "fft_stride_DY")
    # cgemm with beta (M = 64*S: 64 and 320 exercise the partly filled last block of 256 rows)
    A32 = A_ref.astype(np.complex64).reshape(K, M)
    rng = np.random.default_rng(3)
    C0 = (rng.uniform(-1, 1, (N, M)) + 1j * rng.uniform(-1, 1, (N, M))).astype(np.complex64)
    C = dev(C0.copy())
    tf.cgemm(M, N, K, dev(A32), dev(W), C, alpha, beta)
    torch.cuda.synchronize()
    check(C, oracle.cgemm(A32, W, alpha) + beta * C0.astype(np.complex128), tol, "cgemm beta")
    # variant B: fused FFT + CGEMM with beta
    C = dev(C0.copy())
    tf.fused_fft_cgemm(M, N, K, dev(x), dev(W), C, alpha, beta)
    torch.cuda.synchronize()
    C_ref = oracle.cgemm(A_ref.reshape(K, M), W, alpha) + beta * C0.astype(np.complex128)
    check(C, C_ref, tol, "fused_fft_cgemm")
    # backward stage of A and B: [N*S][64] -> [N*S][DY]
    Cin = C_ref.astype(np.complex64).reshape(N, S, 64)
    y = torch.empty((N, S, DY), dtype=torch.complex64, device="cuda")
    tf.ifft_stride_DY(dev(Cin), y, 4, N * S)
    torch.cuda.synchronize()
    check(y, oracle.ifft_pad_contig(Cin.astype(np.complex128), DY), tol, "ifft_stride_DY")
    # variant C: CGEMM + iFFT from the A matrix
    y = torch.empty((N, S, DY), dtype=torch.complex64, device="cuda")
    tf.fused_cgemm_ifft(M, N, K, dev(A32), dev(W), y, alpha)
    torch.cuda.synchronize()
    ref = oracle.ifft_pad_contig(oracle.cgemm(A32, W, alpha).reshape(N, S, 64), DY)
    check(y, ref, tol, "fused_cgemm_ifft")


@pytest.mark.parametrize("DX,DY", [(256, 256), (128, 256), (256, 128), (128, 128), (256, 512), (128, 1024)])
def test_image_stage_entry_points(DX, DY, tol):
    """turbofno_fft2d_trunc / turbofno_ifft2d_pad on their own, through the documented order of the 4096 retained
    modes: element mm*(64*LX) + q*LX + t holds mode (p = t + LX*mm, q), LX = DX/16"""
    print("case image stages", DX, DY, flush=True)
    nimg, LX = 3, DX // 16
    rng = np.random.default_rng(DX * 3 + DY)
    x = (rng.uniform(-1, 1, (nimg, DX, DY)) + 1j * rng.uniform(-1, 1, (nimg, DX, DY))).astype(np.complex64)
    e = np.arange(4096)
    mm, q, t = e // (64 * LX), (e % (64 * LX)) // LX, e % LX
    p = t + LX * mm
    spec = torch.empty((nimg, 4096), dtype=torch.complex64, device="cuda")
    tf.fft2d_trunc(dev(x), spec)
    torch.cuda.synchronize()
    full = np.fft.fft2(x.astype(np.complex128), axes=(1, 2))
    check(spec, full[:, p, q], tol, "fft2d_trunc")
    modes = (rng.uniform(-1, 1, (nimg, 64, 64)) + 1j * rng.uniform(-1, 1, (nimg, 64, 64))).astype(np.complex64)
    y = torch.empty((nimg, DX, DY), dtype=torch.complex64, device="cuda")
    tf.ifft2d_pad(dev(modes[:, p, q]), y)
    torch.cuda.synchronize()
    padded = np.zeros((nimg, DX, DY), dtype=np.complex128)
    padded[:, :64, :64] = modes
    check(y, np.fft.ifft2(padded, axes=(1, 2)) * (DX * DY), tol, "ifft2d_pad")


# (S, DY, K, N, kernel the size rule picks on 256 CUs without an exchange buffer): one shape per branch of the rule
SIZE_RULE_SHAPES = [
    (1, 128, 8, 64, 4), (40, 256, 24, 128, 4),        # at most one 32-channel tile per CU: 512 threads, tiles of 32
    (200, 128, 16, 64, 2), (200, 256, 40, 64, 2),     # up to one 64-channel item per CU: 512 threads
    (300, 256, 32, 64, 3), (700, 256, 8, 64, 3),      # several items per CU: 256 threads
    (300, 128, 32, 64, 8), (800, 128, 64, 128, 8),    # DY = 128: wide tiles
    (1000, 256, 16, 128, 8), (300, 256, 128, 64, 8),   # DY = 256: tiles of 128 channels / 128 input channels
    (1100, 128, 24, 64, 5), (600, 128, 8, 64, 5),     # DY = 128, several items per SIMD: one wavefront per item
    (64, 256, 64, 128, 6), (100, 256, 96, 64, 6),     # small grids, 64 channels or more: K split over the waves of a block
    (100, 512, 16, 64, 2), (300, 512, 16, 64, 1), (300, 1024, 64, 64, 3),   # the long lengths
]


@pytest.mark.parametrize("S,DY,K,N,kernel", SIZE_RULE_SHAPES)
def test_layer_1d_size_rule_against_oracle(S, DY, K, N, kernel, tol):
    """the kernel chosen by size, asserted through the query and checked against the oracle: one shape for every branch of
    the rule (the clustered kernel, which needs an exchange buffer, has its own tests)"""
    print("case size rule vs oracle", S, DY, K, N, "kernel", kernel, flush=True)
    if torch.cuda.get_device_properties(0).multi_processor_count == 256:
        assert tf.query_1d_kernel(DY, S, N, K, compute_units=0) == kernel
    x, W = workloads.uniform_1d(7000 + S + DY + K + N, S, DY, K, N)
    y = tf.layer_1d(dev(x), dev(W), alpha=0.5 - 0.75j)
    torch.cuda.synchronize()
    check(y, oracle.layer_1d(x, W, 0.5 - 0.75j), tol, "size rule S=%d DY=%d K=%d N=%d" % (S, DY, K, N))


def test_layer_1d_across_the_size_rule():
    """60 seeded shapes from one signal set to a few items per CU (S up to 700, all four lengths, K up to 136, N up to
    256), kernel chosen by size: crosses every branch of the choice (clustered, 512- and 256-thread blocks, one
    wavefront per item, SIMT for the long lengths). The oracle takes minutes at these sizes, so the comparison is with
    an fp64 evaluation of the same definition by torch.fft / einsum on the GPU (the oracle itself is pinned to
    numpy.fft and covers the small shapes above)."""
    rng = np.random.default_rng(20251)
    gen = torch.Generator(device="cuda").manual_seed(7)
    for it in range(60):
        DY = int(rng.choice([128, 256, 256, 256, 512, 1024]))
        K = 8 * int(rng.integers(1, 18))
        N = 64 * int(rng.integers(1, 5)) if rng.random() < 0.3 else int(rng.choice([64, 128]))
        S = int(rng.integers(1, 700)) if rng.random() < 0.5 else int(rng.integers(1, 70))
        if DY >= 512:
            S = min(S, 200)
        alpha = complex(rng.uniform(-1, 1), rng.uniform(-1, 1))
        print("case size rule", it, "S", S, "DY", DY, "K", K, "N", N, flush=True)
        x = torch.complex(torch.rand((K, S, DY), generator=gen, device="cuda") - 0.5,
                          torch.rand((K, S, DY), generator=gen, device="cuda") - 0.5)
        W = torch.complex(torch.rand((N, K), generator=gen, device="cuda") - 0.5,
                          torch.rand((N, K), generator=gen, device="cuda") - 0.5)
        y = tf.layer_1d(x, W, alpha=alpha).to(torch.complex128)
        spec = torch.fft.fft(x.to(torch.complex128), dim=-1)[..., :64]
        padded = torch.zeros((N, S, DY), dtype=torch.complex128, device="cuda")
        padded[..., :64] = alpha * torch.einsum("ksm,nk->nsm", spec, W.to(torch.complex128))
        ref = torch.fft.ifft(padded, dim=-1) * DY                    # unnormalised backward transform
        err = float(torch.linalg.vector_norm(y - ref) / torch.linalg.vector_norm(ref))
        worst = float((y - ref).abs().max() / ref.abs().max())
        assert err <= 1e-5 and worst <= 1e-4, (it, S, DY, K, N, err, worst)
