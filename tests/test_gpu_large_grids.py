"""Grids beyond 65,536 blocks on every kernel that indexes a one-dimensional grid (the reference needs a 2D grid
there, fusion_variants_benchmark/2D_D_exp_fused_fft_cgemm_ifft/fused_trunc_2D.cu:172-177, and its default problem
list sweeps the batch to 32,768: benchmark_config/problem_size_1d.txt:1). The full-size result stays on the GPU; a
handful of signals - the first ones, both sides of the 65,535 / 65,536 boundary, the tail of the XCD-aware block
decode, the last ones - are compared with the oracle on those slices only."""
import numpy as np
import pytest
import torch

import oracle
import turbofno_amd as tf
from conftest import max_rel, max_rel_elementwise, rel_l2

pytestmark = pytest.mark.gpu


def _uniform(gen, shape):
    """complex64 uniform[-1,1] generated on the GPU (seeded), so that gigabyte inputs need no host copy"""
    re = torch.rand(shape, generator=gen, device="cuda", dtype=torch.float32) * 2 - 1
    im = torch.rand(shape, generator=gen, device="cuda", dtype=torch.float32) * 2 - 1
    return torch.complex(re, im)


def _check(got, ref, tol, what):
    e2, em, ee = rel_l2(got, ref), max_rel(got, ref), max_rel_elementwise(got, ref)
    print("%s rel_l2=%.3e max_rel=%.3e elementwise=%.3e" % (what, e2, em, ee), flush=True)
    assert e2 <= tol["l2"] and em <= tol["max"] and ee <= tol["elem"], (what, e2, em, ee)


@pytest.mark.parametrize("S,DY,K,N,algo", [
    (40003, 128, 8, 128, 0),         # 80,006 blocks, S odd: exercises the tail of the block decode
    (33001, 256, 8, 128, 0),         # 66,002 blocks at DY = 256
    (66000, 128, 16, 64, 1),         # SIMT kernel, 66,000 blocks
    (33000, 256, 32, 128, 3),        # 256-thread matrix-core kernel, 66,000 blocks
])
def test_layer_1d_beyond_65536_blocks(S, DY, K, N, algo, tol, algo_1d):
    print("large grid layer_1d", S, DY, K, N, algo, flush=True)
    gen = torch.Generator(device="cuda").manual_seed(S + K)
    x = _uniform(gen, (K, S, DY))
    W = _uniform(gen, (N, K)) / np.sqrt(K)
    algo_1d(algo)
    y = tf.layer_1d(x, W, alpha=1 - 1j)
    torch.cuda.synchronize()
    per_tile = 65536 // (N // 64)
    picks = {0, 1, 7, 8, per_tile - 1, per_tile, per_tile + 1, S // 2, (S // 8) * 8 - 1, (S // 8) * 8, S - 2, S - 1}
    picks = sorted(p for p in picks if 0 <= p < S)      # (S // 8) * 8 == S when S is a multiple of 8
    idx = torch.tensor(picks, device="cuda")
    xs = x.index_select(1, idx).cpu().numpy()
    ref = oracle.layer_1d(xs, W.cpu().numpy(), 1 - 1j)
    _check(y.index_select(1, idx).cpu().numpy(), ref, tol, "layer_1d S=%d" % S)


@pytest.mark.parametrize("S,DY,K,N,algo", [
    (2048, 256, 8, 128, 0),          # 4 MiB between the rows of a signal set, two output tiles per set
    (4096, 256, 16, 64, 3),          # 8 MiB, 256-thread matrix-core kernel
    (4096, 128, 16, 64, 5),          # 4 MiB, one wavefront per item
    (1024, 512, 8, 128, 0),          # 4 MiB at length 512
    (512, 1024, 8, 64, 1),           # 4 MiB at length 1024, SIMT kernel
    (2048, 256, 32, 256, 8),         # wide tiles, two per signal set
    (2048, 256, 64, 64, 6),          # eight waves split the channels of an item, two 32-channel tiles per signal set
    (2048, 256, 64, 128, 2),         # 512-thread matrix-core kernel
    (8192, 256, 8, 64, 0),           # 16 MiB: the largest stride that takes this block order
    (16384, 256, 8, 64, 0),          # 32 MiB: back to the interleaved order
])
def test_layer_1d_channel_strides_that_are_multiples_of_4MiB(S, DY, K, N, algo, tol, algo_1d):
    """batch sizes for which XCD j walks the j-th eighth of the signal sets instead of every eighth set: every row of y
    is written (y starts as NaN), and the sets at the seams of the eighths agree with the oracle"""
    print("power-of-two stride layer_1d", S, DY, K, N, algo, flush=True)
    gen = torch.Generator(device="cuda").manual_seed(S + DY + K)
    x = _uniform(gen, (K, S, DY))
    W = _uniform(gen, (N, K)) / np.sqrt(K)
    y = torch.full((N, S, DY), float("nan"), dtype=torch.complex64, device="cuda")
    algo_1d(algo)
    tf.layer_1d(x, W, y=y, alpha=0.5 + 1j)
    torch.cuda.synchronize()
    assert not bool(torch.isnan(torch.view_as_real(y)).any()), "rows of y left unwritten"
    e = S // 8
    picks = sorted({0, 1, 7, 8, e - 1, e, e + 1, 3 * e - 1, 3 * e, S // 2, 7 * e - 1, 7 * e, S - 2, S - 1})
    idx = torch.tensor(picks, device="cuda")
    ref = oracle.layer_1d(x.index_select(1, idx).cpu().numpy(), W.cpu().numpy(), 0.5 + 1j)
    _check(y.index_select(1, idx).cpu().numpy(), ref, tol, "layer_1d S=%d DY=%d" % (S, DY))


@pytest.mark.parametrize("M,K,N,beta", [
    (131072, 64, 64, 0.0),           # 512 column blocks: two per CU, the walk in eighths
    (131072 + 192, 24, 128, 0.0),    # a partly filled last column block, two n tiles, 513 column blocks (plain walk)
    (262144, 40, 64, 0.0),           # four per CU
    (65536, 64, 128, 0.0),           # two n tiles share the CUs: 128 blocks per n tile, two column blocks each
    (65536 + 64, 48, 192, 0.0),      # three n tiles, a partly filled last column block
    (262144, 104, 128, 0.0),         # more than 64 channels, eight column blocks per CU: the whole W tile in LDS, chunks of 32
    (524288 + 128, 72, 64, 0.0),     # the same with one n tile and a partly filled last column block
    (262144, 40, 64, 0.25 - 0.5j),   # C read and written (beta): the kernel with one column block per block
])
def test_cgemm_with_several_column_blocks_per_cu(M, K, N, beta, tol):
    """the mode GEMM as persistent blocks that walk the column blocks: every column written (C starts as NaN when beta
    is zero), columns at the start, at the seams of the eighths and at the end against the oracle"""
    print("persistent cgemm", M, K, N, beta, flush=True)
    gen = torch.Generator(device="cuda").manual_seed(M + K)
    A = _uniform(gen, (K, M))
    W = _uniform(gen, (N, K)) / np.sqrt(K)
    C0 = _uniform(gen, (N, M)) if beta != 0.0 else torch.full((N, M), float("nan"), dtype=torch.complex64, device="cuda")
    C = C0.clone()
    tf.cgemm(M, N, K, A, W, C, 0.5 + 1j, beta)
    torch.cuda.synchronize()
    assert not bool(torch.isnan(torch.view_as_real(C)).any()), "columns of C left unwritten"
    seam = (M // 256 // 8) * 256
    picks = sorted(set(list(range(0, 40)) + list(range(seam - 20, seam + 20)) + list(range(5 * seam - 20, 5 * seam + 20))
                       + list(range(M // 2, M // 2 + 16)) + list(range(M - 300, M))))
    idx = torch.tensor(picks, device="cuda")
    ref = oracle.cgemm(A.index_select(1, idx).cpu().numpy(), W.cpu().numpy(), 0.5 + 1j)
    if beta != 0.0:
        ref = ref + beta * C0.index_select(1, idx).cpu().numpy().astype(np.complex128)
    _check(C.index_select(1, idx).cpu().numpy(), ref, tol, "cgemm M=%d K=%d N=%d" % (M, K, N))


@pytest.mark.parametrize("DX,DY,nsig", [(128, 256, 8300), (256, 128, 16500)])
def test_stride_kernels_beyond_65536_blocks(DX, DY, nsig, tol):
    """X-axis kernels: nsig * DY / 16 (forward) and nsig * DY / 32 (backward) blocks, both above 65,536"""
    print("large grid stride", DX, DY, nsig, flush=True)
    gen = torch.Generator(device="cuda").manual_seed(DX + nsig)
    x = _uniform(gen, (nsig, DX, DY))
    t1 = torch.empty((nsig, 64, DY), dtype=torch.complex64, device="cuda")
    tf.fft_stride(x, t1, 4, DY, DY * nsig, 64)
    back = torch.empty((nsig, DX, DY), dtype=torch.complex64, device="cuda")
    tf.ifft_stride(t1, back, 4, DY, DY * nsig, 64)
    torch.cuda.synchronize()
    cols_fwd, cols_bwd = 65536 * 16 // DY, 65536 * 32 // DY          # signal that holds block 65,536 of either kernel
    assert cols_bwd < nsig
    picks = sorted({0, 1, cols_fwd - 1, cols_fwd, cols_bwd - 1, cols_bwd, nsig // 2, nsig - 1})
    idx = torch.tensor(picks, device="cuda")
    t1_ref = oracle.fft_stride(x.index_select(0, idx).cpu().numpy())
    _check(t1.index_select(0, idx).cpu().numpy(), t1_ref, tol, "fft_stride nsig=%d" % nsig)
    t1_in = t1.index_select(0, idx).cpu().numpy()
    _check(back.index_select(0, idx).cpu().numpy(), oracle.ifft_stride(t1_in.astype(np.complex128), DX), tol,
           "ifft_stride nsig=%d" % nsig)


@pytest.mark.parametrize("DY,nsig", [(128, 2100001), (256, 1050003)])
def test_stride_DY_kernels_beyond_65536_blocks(DY, nsig, tol):
    """contiguous transforms of variant A: 256 / (DY / 16) signals per block, 65,626 blocks, odd signal counts"""
    print("large grid stride_DY", DY, nsig, flush=True)
    gen = torch.Generator(device="cuda").manual_seed(DY + nsig)
    x = _uniform(gen, (nsig, DY))
    A = torch.empty((nsig, 64), dtype=torch.complex64, device="cuda")
    tf.fft_stride_DY(x, A, 4, nsig)
    y = torch.empty((nsig, DY), dtype=torch.complex64, device="cuda")
    tf.ifft_stride_DY(A, y, 4, nsig)
    torch.cuda.synchronize()
    per_block = 256 // (DY // 16)
    assert 65536 * per_block < nsig
    picks = sorted({0, 1, 65535 * per_block, 65536 * per_block - 1, 65536 * per_block, nsig // 2, nsig - 2, nsig - 1})
    idx = torch.tensor(picks, device="cuda")
    A_ref = oracle.fft_trunc_contig(x.index_select(0, idx).cpu().numpy())
    _check(A.index_select(0, idx).cpu().numpy(), A_ref, tol, "fft_stride_DY nsig=%d" % nsig)
    A_in = A.index_select(0, idx).cpu().numpy()
    _check(y.index_select(0, idx).cpu().numpy(), oracle.ifft_pad_contig(A_in.astype(np.complex128), DY), tol,
           "ifft_stride_DY nsig=%d" % nsig)


def test_cgemm_beyond_65536_rows_per_channel(tol):
    """mode-space GEMM with M = 2^24 rows: 65,536 blocks of 256 rows"""
    M, N, K = 1 << 24, 64, 8
    print("large grid cgemm", M, N, K, flush=True)
    gen = torch.Generator(device="cuda").manual_seed(77)
    A = _uniform(gen, (K, M))
    W = _uniform(gen, (N, K))
    C = torch.empty((N, M), dtype=torch.complex64, device="cuda")
    tf.cgemm(M, N, K, A, W, C, 1 - 1j, 0.0)
    torch.cuda.synchronize()
    picks = torch.tensor(sorted({0, 255, 256, 65535 * 256 - 1, 65535 * 256, M // 2 + 3, M - 257, M - 1}), device="cuda")
    ref = oracle.cgemm(A.index_select(1, picks).cpu().numpy(), W.cpu().numpy(), 1 - 1j)
    _check(C.index_select(1, picks).cpu().numpy(), ref, tol, "cgemm M=2^24")


def test_row_kernels_beyond_65536_blocks(tol):
    """2D layer with whole rows first on 66 x 8 input and 66 x 64 output images of 512 x 512: the backward row kernel runs
    67,584 blocks (one per 32 rows), the forward row kernel walks 8,448 row blocks with its persistent grid; batch
    elements on both sides of block 65,536 and the last one against the oracle"""
    bs, D, K, N = 66, 512, 8, 64
    print("large grid rows first", bs, D, K, N, flush=True)
    gen = torch.Generator(device="cuda").manual_seed(91)
    x = _uniform(gen, (K, bs, D, D))
    W = _uniform(gen, (N, K))
    y = tf.layer_2d(x, W, alpha=1 - 1j, algo=3)
    torch.cuda.synchronize()
    assert N * bs * (D // 32) > 65536
    # output image n * bs + b is written by blocks 16 (n * bs + b) ... + 15: block 65,536 lies in image 4096 = (n 62, b 4)
    for b in (0, 3, 4, 65):
        ref = oracle.layer_2d(x[:, b:b + 1].cpu().numpy(), W.cpu().numpy(), 1 - 1j)
        _check(y[:, b:b + 1].cpu().numpy(), ref, tol, "rows first bs=66 b=%d" % b)
