"""The entry points allocate nothing, never synchronise and record no memset nodes, so a caller can capture them in a
HIP graph. Each captured layer is replayed several times, with eager work and synchronisations between the replays and
fresh input written into the captured buffers, and every replay is compared with the eager result."""
import numpy as np
import pytest
import torch

import turbofno_amd as tf
from turbofno_amd import workloads

pytestmark = pytest.mark.gpu


def _rel(a, b):
    return float(torch.linalg.vector_norm(a - b) / torch.linalg.vector_norm(b))


@pytest.mark.parametrize("algo", [1, 2, 3])
def test_layer_2d_in_a_graph(algo):
    print("graph 2d algo", algo, flush=True)
    bs, D, K, N = 4, 128, 64, 64
    xs = [torch.from_numpy(workloads.uniform_2d(900 + i, bs, D, D, K, N)[0]).cuda() for i in range(3)]
    W = torch.from_numpy(workloads.uniform_2d(900, bs, D, D, K, N)[1]).cuda()
    x = xs[0].clone()
    y = torch.empty((N, bs, D, D), dtype=torch.complex64, device="cuda")
    ws = torch.empty(tf.layer_2d_workspace_bytes(bs, D, D, K, N, algo), dtype=torch.uint8, device="cuda")
    tf.layer_2d(x, W, y=y, workspace=ws, algo=algo)          # first launch outside the capture (kernel attributes)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        tf.layer_2d(x, W, y=y, workspace=ws, algo=algo)
    for i in (1, 2, 0, 1):
        x.copy_(xs[i])
        expect = tf.layer_2d(xs[i], W, algo=algo)            # eager, own buffers
        torch.cuda.synchronize()
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert _rel(y, expect) == 0.0, (i, _rel(y, expect))


@pytest.mark.parametrize("K", [16, 128])
def test_layer_1d_in_a_graph(K):
    print("graph 1d K", K, flush=True)
    bs, DY, N = 64, 256, 128
    xs = [torch.from_numpy(workloads.smooth_1d(950 + i, bs, DY, K, N)[0]).cuda() for i in range(3)]
    W = torch.from_numpy(workloads.smooth_1d(950, bs, DY, K, N)[1]).cuda()
    x = xs[0].clone()
    y = torch.empty((N, bs, DY), dtype=torch.complex64, device="cuda")
    # warm-up on the stream that is captured afterwards (raises the kernels' dynamic-LDS limits outside the capture)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        tf.layer_1d(x, W, y=y)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        tf.layer_1d(x, W, y=y)
    for i in (2, 1, 0):
        x.copy_(xs[i])
        expect = tf.layer_1d(xs[i], W)
        torch.cuda.synchronize()
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert _rel(y, expect) == 0.0, (i, _rel(y, expect))
