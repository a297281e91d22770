"""The clustered fused 1D kernel (small grids, K >= 64, DY = 256, N in {64, 128}): several blocks share a signal set,
split its K channels and exchange partial products through a library-owned device buffer. Checked against the CPU
oracle on the shapes that select each cluster size and chunk size, across repeated launches (the arrival counters are
never reset), on two streams at once (separate buffers), from a replayed graph, and on the error path of a wait that
gives up."""
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


def check(got, ref, tol, what):
    got = got.cpu().numpy()
    e2, em, ee = rel_l2(got, ref), max_rel(got, ref), max_rel_elementwise(got, ref)
    print("%s rel_l2=%.3e max_rel=%.3e elementwise=%.3e" % (what, e2, em, ee), flush=True)
    assert e2 <= tol["l2"] and em <= tol["max"] and ee <= tol["elem"], (what, e2, em, ee)


# S, K, N -> cluster size / channels per member / chunk (on 256 CUs)
SHAPES = [
    (64, 128, 128),   # the large-hidden benchmark case: 4 members x 32 channels, one chunk of 32
    (64, 64, 128),    # 4 x 16, chunk 16
    (32, 128, 128),   # 8 members x 16 channels, 16 output channels each
    (13, 64, 128),    # S not a multiple of 8: padding blocks of the last group of clusters leave at once
    (64, 64, 64),     # N = 64: 4 members own 16 output channels each
    (33, 128, 64),    # 40 cluster slots x 4
    (3, 256, 128),    # 8 x 32
    (64, 256, 128),   # 4 x 64: two chunks per member, accumulators kept across them
    (5, 192, 64),     # 8 x 24: chunk 8, three chunks
    (128, 64, 64),    # 2 members x 32 channels, 32 output channels each
    (1, 64, 64),
]


@pytest.mark.parametrize("algo", [0, 7])
@pytest.mark.parametrize("S,K,N", SHAPES)
def test_cluster_against_oracle(S, K, N, algo, tol, algo_1d):
    print("case cluster", S, K, N, "algo", algo, flush=True)
    algo_1d(algo)
    x, W = workloads.uniform_1d(300 + S + K + N, S, 256, K, N)
    ref = oracle.layer_1d(x, W, 0.75 - 0.5j)
    xd, Wd = dev(x), dev(W)
    for rep in range(3):            # the counters of a stream keep counting from launch to launch
        y = tf.layer_1d(xd, Wd, alpha=0.75 - 0.5j)
        torch.cuda.synchronize()
        check(y, ref, tol, "cluster S=%d K=%d N=%d launch %d" % (S, K, N, rep))


def test_cluster_matches_block_kernel_on_the_large_hidden_case(tol, algo_1d):
    """bs = 64, DY = 256, K = N = 128 with the generator the benchmark uses: clustered kernel against the kernel that
    keeps a signal set inside one block (no exchange), element by element"""
    print("case cluster vs block kernel", flush=True)
    x, W = workloads.smooth_1d(5, 64, 256, 128, 128)
    xd, Wd = dev(x), dev(W)
    algo_1d(2)
    ref = tf.layer_1d(xd, Wd).cpu().numpy()
    algo_1d(7)
    check(tf.layer_1d(xd, Wd), ref, tol, "cluster vs block kernel")


def test_cluster_on_two_streams(tol, algo_1d):
    """launches on two streams overlap on the GPU; each stream has its own exchange buffer"""
    print("case cluster two streams", flush=True)
    algo_1d(7)
    S, K, N = 24, 128, 128
    probs = []
    for i in range(2):
        x, W = workloads.uniform_1d(900 + i, S, 256, K, N)
        probs.append((dev(x), dev(W), oracle.layer_1d(x, W, 1.0), torch.empty((N, S, 256), dtype=torch.complex64, device="cuda")))
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    for _ in range(20):
        for (xd, Wd, _, y), st in zip(probs, streams):
            with torch.cuda.stream(st):
                tf.layer_1d(xd, Wd, y=y)
    torch.cuda.synchronize()
    for i, (_, _, ref, y) in enumerate(probs):
        check(y, ref, tol, "cluster stream %d" % i)


def test_cluster_in_a_replayed_graph(tol, algo_1d):
    """captured after a first eager call (which allocates the stream's buffer); every replay is checked, with eager
    launches on the same stream in between"""
    print("case cluster graph", flush=True)
    algo_1d(7)
    S, K, N = 64, 128, 128
    x, W = workloads.uniform_1d(77, S, 256, K, N)
    ref = oracle.layer_1d(x, W, 1.0)
    xd, Wd = dev(x), dev(W)
    y = torch.empty((N, S, 256), dtype=torch.complex64, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        tf.layer_1d(xd, Wd, y=y)                    # allocates the exchange buffer of this stream
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            tf.layer_1d(xd, Wd, y=y)
        for rep in range(4):
            y.fill_(0)
            graph.replay()
            side.synchronize()
            check(y, ref, tol, "cluster graph replay %d" % rep)
            y2 = tf.layer_1d(xd, Wd)                # eager launch between replays, same stream
            side.synchronize()
            check(y2, ref, tol, "cluster eager after replay %d" % rep)


def test_cluster_wait_that_gives_up_is_reported(tol, algo_1d):
    """with a wait bound of zero every block that has to wait gives up (all kernels still run to completion); the next
    call on the stream reports it once, the one after that works again"""
    print("case cluster gives up", flush=True)
    algo_1d(7)
    S, K, N = 64, 128, 128
    x, W = workloads.uniform_1d(78, S, 256, K, N)
    xd, Wd = dev(x), dev(W)
    tf.layer_1d(xd, Wd)
    torch.cuda.synchronize()
    tf.set_exchange_wait_us(0)
    try:
        tf.layer_1d(xd, Wd)                         # output invalid
        torch.cuda.synchronize()
    finally:
        tf.set_exchange_wait_us(2_000_000)
    with pytest.raises(tf.TurboFNOError) as err:
        tf.layer_1d(xd, Wd)
    assert err.value.code == 5, err.value
    y = tf.layer_1d(xd, Wd)
    torch.cuda.synchronize()
    check(y, oracle.layer_1d(x, W, 1.0), tol, "cluster after a reported give-up")
