"""The clustered fused 1D kernel (small grids, K >= 64, DY = 256, N in {64, 128}): several blocks share a signal set,
split its K channels and exchange partial products through a CALLER-owned device buffer that is attached to a stream.
Checked against the CPU oracle on the shapes that select each cluster size and chunk size, across repeated launches (the
arrival counters are never reset), on two streams at once (one buffer each), from a replayed graph, and with a wait
bound of zero, where every member that would have to wait computes the other members' share itself: the output stays
valid and the event is counted. Without an attached buffer the library must neither allocate nor take this kernel."""
import ctypes

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


@pytest.fixture
def exchange():
    """an exchange buffer attached to torch's current stream for the duration of one test"""
    with tf.ExchangeBuffer() as ex:
        yield ex


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
def test_cluster_against_oracle(S, K, N, algo, tol, algo_1d, exchange):
    print("case cluster", S, K, N, "algo", algo, flush=True)
    algo_1d(algo, attach=False)
    assert tf.query_1d_kernel(256, S, N, K, compute_units=0, exchange_attached=True) == 7
    x, W = workloads.uniform_1d(300 + S + K + N, S, 256, K, N)
    ref = oracle.layer_1d(x, W, 0.75 - 0.5j)
    xd, Wd = dev(x), dev(W)
    for rep in range(3):            # the counters of a stream keep counting from launch to launch
        y = tf.layer_1d(xd, Wd, alpha=0.75 - 0.5j)
        torch.cuda.synchronize()
        check(y, ref, tol, "cluster S=%d K=%d N=%d launch %d" % (S, K, N, rep))
    # (members that start late, as on the first launch after an idle period, may have used the fallback: still valid)


def test_cluster_matches_block_kernel_on_the_large_hidden_case(tol, algo_1d, exchange):
    """bs = 64, DY = 256, K = N = 128 with the generator the benchmark uses: clustered kernel against the kernel that
    keeps a signal set inside one block (no exchange), element by element"""
    print("case cluster vs block kernel", flush=True)
    x, W = workloads.smooth_1d(5, 64, 256, 128, 128)
    xd, Wd = dev(x), dev(W)
    algo_1d(2)
    ref = tf.layer_1d(xd, Wd).cpu().numpy()
    algo_1d(7, attach=False)
    check(tf.layer_1d(xd, Wd), ref, tol, "cluster vs block kernel")


def test_without_a_buffer_nothing_is_allocated_and_another_kernel_runs(tol, algo_1d):
    """no exchange buffer attached: the choice by size (and the forced selector 7) fall back on the kernel that splits
    K inside one block, and the call leaves the free device memory exactly as it found it"""
    print("case no buffer", flush=True)
    S, K, N = 64, 128, 128
    assert tf.query_1d_kernel(256, S, N, K, compute_units=0, exchange_attached=False) == 6
    x, W = workloads.uniform_1d(41, S, 256, K, N)
    ref = oracle.layer_1d(x, W, 1.0)
    xd, Wd = dev(x), dev(W)
    y = torch.empty((N, S, 256), dtype=torch.complex64, device="cuda")
    tf.layer_1d(xd, Wd, y=y)                    # the HIP runtime's own first-launch work for this kernel happens here
    side = torch.cuda.Stream()                  # a stream the library has never seen;
    with torch.cuda.stream(side):
        y.zero_()                               # ... and the runtime's per-stream set-up here
    torch.cuda.synchronize()
    for algo in (0, 7):
        algo_1d(algo, attach=False)
        free_before = torch.cuda.mem_get_info()[0]
        with torch.cuda.stream(side):
            tf.layer_1d(xd, Wd, y=y)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "the 1D layer call changed the free device memory"
        check(y, ref, tol, "no buffer, selector %d" % algo)


def test_cluster_on_two_streams(tol, algo_1d):
    """launches on two streams overlap on the GPU; each stream has its own exchange buffer"""
    print("case cluster two streams", flush=True)
    algo_1d(7, attach=False)
    S, K, N = 24, 128, 128
    probs = []
    for i in range(2):
        x, W = workloads.uniform_1d(900 + i, S, 256, K, N)
        probs.append((dev(x), dev(W), oracle.layer_1d(x, W, 1.0), torch.empty((N, S, 256), dtype=torch.complex64, device="cuda")))
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    buffers = [tf.ExchangeBuffer(stream=st) for st in streams]
    torch.cuda.synchronize()
    try:
        for _ in range(20):
            for (xd, Wd, _, y), st in zip(probs, streams):
                with torch.cuda.stream(st):
                    tf.layer_1d(xd, Wd, y=y)
        torch.cuda.synchronize()
    finally:
        for b in buffers:
            b.close()
    for i, (_, _, ref, y) in enumerate(probs):
        check(y, ref, tol, "cluster stream %d" % i)


def test_cluster_in_a_replayed_graph(tol, algo_1d):
    """the buffer is attached before the capture; every replay is checked, with eager launches on the same stream in
    between (they share the stream's buffer and its counters)"""
    print("case cluster graph", flush=True)
    algo_1d(7, attach=False)
    S, K, N = 64, 128, 128
    x, W = workloads.uniform_1d(77, S, 256, K, N)
    ref = oracle.layer_1d(x, W, 1.0)
    xd, Wd = dev(x), dev(W)
    y = torch.empty((N, S, 256), dtype=torch.complex64, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side), tf.ExchangeBuffer(stream=side):
        tf.layer_1d(xd, Wd, y=y)
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


@pytest.mark.parametrize("S,K,N,P", [(64, 128, 128, 4), (5, 192, 64, 8), (128, 64, 64, 2)])
def test_cluster_members_that_work_alone_still_deliver(S, K, N, P, tol, algo_1d, exchange):
    """with a wait bound of zero no member waits for the others: each computes the other members' share itself (all
    kernels run to completion), the output is valid, and every member counts itself in the buffer, where the status call
    finds the number once; the launches after that exchange partial products as before"""
    print("case cluster members work alone", S, K, N, flush=True)
    algo_1d(7, attach=False)
    x, W = workloads.uniform_1d(78 + S, S, 256, K, N)
    ref = oracle.layer_1d(x, W, 0.5 + 0.25j)
    xd, Wd = dev(x), dev(W)
    tf.layer_1d(xd, Wd, alpha=0.5 + 0.25j)
    exchange.status()
    tf.set_exchange_wait_us(0)
    try:
        for rep in range(2):
            y = tf.layer_1d(xd, Wd, alpha=0.5 + 0.25j)
            torch.cuda.synchronize()
            check(y, ref, tol, "cluster, every member alone, launch %d" % rep)
    finally:
        tf.set_exchange_wait_us(100)
    n = ctypes.c_uint(0)
    rc = tf.lib().turbofno_exchange_status(torch.cuda.current_stream().cuda_stream, ctypes.byref(n))
    assert rc == 5 and n.value == 2 * S * P, (rc, n.value)   # every member of both launches
    assert b"valid" in tf.lib().turbofno_last_error_string()
    assert exchange.status() == 0                            # reported once
    for rep in range(2):                                     # partial products are exchanged again
        y = tf.layer_1d(xd, Wd, alpha=0.5 + 0.25j)
        torch.cuda.synchronize()
        check(y, ref, tol, "cluster after members worked alone, launch %d" % rep)


def test_cluster_launches_of_different_shapes_share_a_buffer(tol, algo_1d, exchange):
    """launches with different cluster sizes and channel counts follow each other on one stream: every word of the buffer
    that a launch used is left ready for whichever launch comes next"""
    print("case cluster mixed shapes", flush=True)
    algo_1d(7, attach=False)
    probs = []
    for i, (S, K, N) in enumerate([(64, 128, 128), (3, 256, 128), (128, 64, 64), (33, 128, 64)]):
        x, W = workloads.uniform_1d(500 + i, S, 256, K, N)
        probs.append((dev(x), dev(W), oracle.layer_1d(x, W, 1.0)))
    for rep in range(3):
        for i in (0, 1, 2, 3, 1, 0, 3, 2):
            xd, Wd, ref = probs[i]
            y = tf.layer_1d(xd, Wd)
            torch.cuda.synchronize()
            check(y, ref, tol, "mixed shapes round %d problem %d" % (rep, i))


def test_cluster_exchange_is_used_on_a_busy_gpu(algo_1d, exchange):
    """back-to-back launches on a GPU that is already running: the members of a cluster start together and exchange
    their partial products; (almost) none falls back on computing the others' share"""
    print("case cluster exchange in use", flush=True)
    algo_1d(7, attach=False)
    S, K, N = 64, 128, 128
    x, W = workloads.uniform_1d(91, S, 256, K, N)
    xd, Wd = dev(x), dev(W)
    y = torch.empty((N, S, 256), dtype=torch.complex64, device="cuda")
    for _ in range(20):
        tf.layer_1d(xd, Wd, y=y)
    exchange.status()
    for _ in range(200):
        tf.layer_1d(xd, Wd, y=y)
    assert exchange.status() <= 4              # of 200 launches x 256 members


def test_attach_refuses_a_buffer_that_is_too_small_or_misaligned():
    L = tf.lib()
    need = tf.exchange_bytes(0)
    assert need == tf.exchange_bytes(torch.cuda.get_device_properties(0).multi_processor_count)
    buf = torch.empty(need + 512, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    assert L.turbofno_exchange_attach(st, buf.data_ptr(), need - 1) == 3
    assert L.turbofno_exchange_attach(st, buf.data_ptr() + 8, need) == 3
    assert L.turbofno_exchange_attach(st, None, need) == 1
    assert L.turbofno_exchange_attach(st, buf.data_ptr(), need) == 0
    assert L.turbofno_exchange_detach(st) == 0
    assert L.turbofno_exchange_detach(st) == 0                          # nothing attached: still fine
    torch.cuda.synchronize()
