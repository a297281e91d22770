"""ctypes binding of the CPU oracle (liboracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the benchmark's
cpu_baseline leg. Nothing in the product package imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

MODES = 64


def build(force=False):
    """Compile liboracle.so with gcc (make). Safe to call repeatedly."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


def _declare(L):
    f32p = ctypes.POINTER(ctypes.c_float)
    f64p = ctypes.POINTER(ctypes.c_double)
    L.oracle_dft_naive.argtypes = [f64p, ctypes.c_long, f64p, ctypes.c_long, ctypes.c_int, ctypes.c_int]
    L.oracle_fft_batched.argtypes = [f64p, ctypes.c_int, ctypes.c_long, ctypes.c_int]
    L.oracle_cgemm.argtypes = [f64p, f64p, f64p, ctypes.c_long, ctypes.c_int, ctypes.c_int,
                               ctypes.c_double, ctypes.c_double]
    L.oracle_fft_trunc_contig.argtypes = [f32p, f64p, ctypes.c_long, ctypes.c_int]
    L.oracle_ifft_pad_contig.argtypes = [f64p, f64p, ctypes.c_long, ctypes.c_int]
    L.oracle_layer_1d.argtypes = [f32p, f32p, f64p, ctypes.c_long, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                  ctypes.c_double, ctypes.c_double]
    L.oracle_fft_stride.argtypes = [f32p, f64p, ctypes.c_long, ctypes.c_int, ctypes.c_int]
    L.oracle_ifft_stride.argtypes = [f64p, f64p, ctypes.c_long, ctypes.c_int, ctypes.c_int]
    L.oracle_layer_2d.argtypes = [f32p, f32p, f64p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                  ctypes.c_int, ctypes.c_double, ctypes.c_double]
    L.cpu_baseline_layer_1d.argtypes = [f32p, f32p, f32p, ctypes.c_long, ctypes.c_int, ctypes.c_int,
                                        ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_int]
    L.cpu_baseline_layer_2d.argtypes = [f32p, f32p, f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                        ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_int]
    L.cpu_baseline_max_threads.restype = ctypes.c_int
    for fn in ("oracle_dft_naive", "oracle_fft_batched", "oracle_cgemm", "oracle_fft_trunc_contig",
               "oracle_ifft_pad_contig", "oracle_layer_1d", "oracle_fft_stride", "oracle_ifft_stride",
               "oracle_layer_2d", "cpu_baseline_layer_1d", "cpu_baseline_layer_2d"):
        getattr(L, fn).restype = None


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.complex64)
    return a, a.view(np.float32).ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _f64(a):
    a = np.ascontiguousarray(a, dtype=np.complex128)
    return a, a.view(np.float64).ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def dft_naive(v, sign):
    """Brute-force O(D^2) DFT of one vector; sign=-1 forward, +1 unnormalised backward."""
    v, vp = _f64(v)
    out = np.empty_like(v)
    lib().oracle_dft_naive(vp, 1, out.view(np.float64).ctypes.data_as(ctypes.POINTER(ctypes.c_double)), 1,
                           v.shape[-1], sign)
    return out


def fft_batched(a, sign):
    a = np.array(a, dtype=np.complex128, order="C", copy=True)
    D = a.shape[-1]
    lib().oracle_fft_batched(a.view(np.float64).ctypes.data_as(ctypes.POINTER(ctypes.c_double)), D,
                             a.size // D, sign)
    return a


def cgemm(A, W, alpha=1.0 + 0j):
    """A: [K][M] (column-major M x K), W: [N][K] (W[k + n*K]) -> C: [N][M]."""
    A, Ap = _f64(A)
    W, Wp = _f64(W)
    K, M = A.shape
    N = W.shape[0]
    C = np.empty((N, M), dtype=np.complex128)
    lib().oracle_cgemm(Ap, Wp, C.view(np.float64).ctypes.data_as(ctypes.POINTER(ctypes.c_double)), M, N, K,
                       complex(alpha).real, complex(alpha).imag)
    return C


def fft_trunc_contig(x):
    x, xp = _f32(x)
    D = x.shape[-1]
    out = np.empty(x.shape[:-1] + (MODES,), dtype=np.complex128)
    lib().oracle_fft_trunc_contig(xp, out.view(np.float64).ctypes.data_as(ctypes.POINTER(ctypes.c_double)),
                                  x.size // D, D)
    return out


def ifft_pad_contig(spec, D):
    spec, sp = _f64(spec)
    out = np.empty(spec.shape[:-1] + (D,), dtype=np.complex128)
    lib().oracle_ifft_pad_contig(sp, out.view(np.float64).ctypes.data_as(ctypes.POINTER(ctypes.c_double)),
                                 spec.size // MODES, D)
    return out


def layer_1d(x, W, alpha=1.0 + 0j):
    """x: [K][S][DY] complex64, W: [N][K] complex64 (element W[k + n*K]) -> y [N][S][DY] complex128."""
    x, xp = _f32(x)
    W, Wp = _f32(W)
    K, S, DY = x.shape
    N = W.shape[0]
    assert W.shape[1] == K
    y = np.empty((N, S, DY), dtype=np.complex128)
    lib().oracle_layer_1d(xp, Wp, y.view(np.float64).ctypes.data_as(ctypes.POINTER(ctypes.c_double)),
                          S, DY, K, N, complex(alpha).real, complex(alpha).imag)
    return y


def fft_stride(x):
    """x: [sig][DX][DY] complex64 -> [sig][64][DY] complex128 (forward along DX, truncated)."""
    x, xp = _f32(x)
    nsig, DX, DY = x.shape
    out = np.empty((nsig, MODES, DY), dtype=np.complex128)
    lib().oracle_fft_stride(xp, out.view(np.float64).ctypes.data_as(ctypes.POINTER(ctypes.c_double)),
                            nsig, DX, DY)
    return out


def ifft_stride(t, DX):
    """t: [sig][64][DY] complex128 -> [sig][DX][DY] complex128 (zero-padded backward along DX)."""
    t, tp = _f64(t)
    nsig, _, DY = t.shape
    out = np.empty((nsig, DX, DY), dtype=np.complex128)
    lib().oracle_ifft_stride(tp, out.view(np.float64).ctypes.data_as(ctypes.POINTER(ctypes.c_double)),
                             nsig, DX, DY)
    return out


def layer_2d(x, W, alpha=1.0 + 0j):
    """x: [K][bs][DX][DY] complex64, W: [N][K] complex64 -> y [N][bs][DX][DY] complex128."""
    x, xp = _f32(x)
    W, Wp = _f32(W)
    K, bs, DX, DY = x.shape
    N = W.shape[0]
    assert W.shape[1] == K
    y = np.empty((N, bs, DX, DY), dtype=np.complex128)
    lib().oracle_layer_2d(xp, Wp, y.view(np.float64).ctypes.data_as(ctypes.POINTER(ctypes.c_double)),
                          bs, DX, DY, K, N, complex(alpha).real, complex(alpha).imag)
    return y


def cpu_baseline_layer_1d(x, W, alpha=1.0 + 0j, nthreads=0):
    x, xp = _f32(x)
    W, Wp = _f32(W)
    K, S, DY = x.shape
    N = W.shape[0]
    y = np.empty((N, S, DY), dtype=np.complex64)
    lib().cpu_baseline_layer_1d(xp, Wp, y.view(np.float32).ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                S, DY, K, N, complex(alpha).real, complex(alpha).imag, nthreads)
    return y


def cpu_baseline_layer_2d(x, W, alpha=1.0 + 0j, nthreads=0):
    x, xp = _f32(x)
    W, Wp = _f32(W)
    K, bs, DX, DY = x.shape
    N = W.shape[0]
    y = np.empty((N, bs, DX, DY), dtype=np.complex64)
    lib().cpu_baseline_layer_2d(xp, Wp, y.view(np.float32).ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                bs, DX, DY, K, N, complex(alpha).real, complex(alpha).imag, nthreads)
    return y


def cpu_threads():
    return int(lib().cpu_baseline_max_threads())
