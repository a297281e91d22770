"""Committed golden vectors (tests/golden/layer_outputs.npz, written by tests/golden/make_golden.py from numpy.fft in
the mix-then-low-pass order): the CPU oracle must reproduce them, and so must the HIP path through the C ABI."""
import importlib.util
import os

import numpy as np
import pytest

import oracle
from conftest import max_rel, rel_l2

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
G = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(G)
GOLD = np.load(os.path.join(HERE, "golden", "layer_outputs.npz"))


def _check(got, want, tol):
    assert got.shape == want.shape
    assert rel_l2(got, want) <= tol["l2"] and max_rel(got, want) <= tol["max"]


@pytest.mark.parametrize("name", sorted(G.CASES_1D))
def test_oracle_matches_golden_1d(name, tol):
    seed, bs, DY, K, N, alpha, ch = G.CASES_1D[name]
    x, W = G.inputs_1d(seed, bs, DY, K, N)
    _check(oracle.layer_1d(x, W, alpha)[list(ch)], GOLD["1d/" + name], tol)


@pytest.mark.parametrize("name", sorted(G.CASES_2D))
def test_oracle_matches_golden_2d(name, tol):
    seed, bs, DX, DY, K, N, alpha, ch, st = G.CASES_2D[name]
    x, W = G.inputs_2d(seed, bs, DX, DY, K, N)
    _check(oracle.layer_2d(x, W, alpha)[list(ch)][..., ::st, ::st], GOLD["2d/" + name], tol)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(G.CASES_1D))
def test_gpu_matches_golden_1d(name, tol):
    import torch
    import turbofno_amd as tf
    seed, bs, DY, K, N, alpha, ch = G.CASES_1D[name]
    x, W = G.inputs_1d(seed, bs, DY, K, N)
    print("golden 1d", name, flush=True)
    y = tf.layer_1d(torch.from_numpy(x).cuda(), torch.from_numpy(W).cuda(), alpha=alpha)
    torch.cuda.synchronize()
    _check(y.cpu().numpy()[list(ch)], GOLD["1d/" + name], tol)


@pytest.mark.gpu
@pytest.mark.parametrize("algo", [1, 2])
@pytest.mark.parametrize("name", sorted(G.CASES_2D))
def test_gpu_matches_golden_2d(name, algo, tol):
    import torch
    import turbofno_amd as tf
    seed, bs, DX, DY, K, N, alpha, ch, st = G.CASES_2D[name]
    x, W = G.inputs_2d(seed, bs, DX, DY, K, N)
    print("golden 2d", name, algo, flush=True)
    y = tf.layer_2d(torch.from_numpy(x).cuda(), torch.from_numpy(W).cuda(), alpha=alpha, algo=algo)
    torch.cuda.synchronize()
    _check(y.cpu().numpy()[list(ch)][..., ::st, ::st], GOLD["2d/" + name], tol)
