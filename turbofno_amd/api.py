"""ctypes binding of libturbofno.so (C ABI: include/turbofno.h).

Function names and argument meaning mirror the reference's kernel tables
(fusion_variants/1D_D_exp_fused_fft_cgemm_ifft/fused.cu:15-16,
fusion_variants/2D_D_exp_fused_fft_cgemm_ifft/fused_trunc_2D.cu:27-30). Tensors are torch
complex64 tensors resident on the GPU; every call is asynchronous on torch's current stream.
"""
import ctypes
import os

import torch

MODES = 64
_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


class TurboFNOError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("turbofno error %d: %s" % (code, message))
        self.code = code


def library_path():
    return os.path.join(_HERE, "libturbofno.so")


def lib():
    """Loads libturbofno.so; raises (no fallback) when it has not been built."""
    global _LIB
    if _LIB is None:
        path = library_path()
        if not os.path.exists(path):
            raise ImportError("%s not found: build it with `make -C turbofno_amd/csrc` "
                              "(or __graft_entry__.build()); there is no fallback path" % path)
        L = ctypes.CDLL(path)
        vp, i, l, f, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float, ctypes.c_size_t
        L.turbofno_fused_fft_cgemm_ifft.argtypes = [i, l, i, i, vp, vp, vp, vp, f, f, f, f, vp]
        L.turbofno_fft_stride.argtypes = [i, vp, vp, i, i, l, i, vp]
        L.turbofno_ifft_stride.argtypes = [i, vp, vp, i, i, l, i, vp]
        L.turbofno_layer_1d.argtypes = [i, i, i, i, i, vp, vp, vp, f, f, vp]
        L.turbofno_layer_2d_workspace_bytes.argtypes = [i, i, i, i, i, i]
        L.turbofno_layer_2d_workspace_bytes.restype = sz
        L.turbofno_layer_2d.argtypes = [i, i, i, i, i, vp, vp, vp, f, f, vp, sz, i, vp]
        L.turbofno_fft2d_trunc.argtypes = [i, i, vp, vp, l, vp]
        L.turbofno_ifft2d_pad.argtypes = [i, i, vp, vp, l, vp]
        L.turbofno_cgemm.argtypes = [l, i, i, vp, vp, vp, f, f, f, f, vp]
        L.turbofno_fft_stride_DY.argtypes = [i, vp, vp, i, l, vp]
        L.turbofno_ifft_stride_DY.argtypes = [i, vp, vp, i, l, vp]
        L.turbofno_fused_fft_cgemm.argtypes = [i, l, i, i, vp, vp, vp, f, f, f, f, vp]
        L.turbofno_fused_cgemm_ifft.argtypes = [i, l, i, i, vp, vp, vp, vp, f, f, f, f, vp]
        L.turbofno_layer_2d_noalloc.argtypes = [i, i, i, i, i, vp, vp, vp, f, f, i, vp]
        L.turbofno_set_1d_algo.argtypes = [i]
        L.turbofno_get_1d_algo.argtypes = []
        L.turbofno_set_exchange_wait_us.argtypes = [ctypes.c_ulonglong]
        L.turbofno_set_exchange_wait_us.restype = i
        L.turbofno_get_1d_algo.restype = i
        L.turbofno_exchange_bytes.argtypes = [i]
        L.turbofno_exchange_bytes.restype = sz
        L.turbofno_exchange_attach.argtypes = [vp, vp, sz]
        L.turbofno_exchange_attach.restype = i
        L.turbofno_exchange_detach.argtypes = [vp]
        L.turbofno_exchange_detach.restype = i
        L.turbofno_exchange_status.argtypes = [vp, ctypes.POINTER(ctypes.c_uint)]
        L.turbofno_exchange_status.restype = i
        L.turbofno_query_2d_algo.argtypes = [i, i, i, i, i, i]
        L.turbofno_query_2d_algo.restype = i
        L.turbofno_query_1d_kernel.argtypes = [i, l, i, i, i, i]
        L.turbofno_query_1d_kernel.restype = i
        L.turbofno_last_error_string.restype = ctypes.c_char_p
        L.turbofno_abi_version.restype = i
        for name in ("turbofno_fused_fft_cgemm_ifft", "turbofno_fft_stride", "turbofno_ifft_stride",
                     "turbofno_layer_1d", "turbofno_layer_2d", "turbofno_fft2d_trunc", "turbofno_ifft2d_pad",
                     "turbofno_cgemm", "turbofno_fft_stride_DY", "turbofno_ifft_stride_DY", "turbofno_fused_fft_cgemm",
                     "turbofno_fused_cgemm_ifft", "turbofno_layer_2d_noalloc", "turbofno_set_1d_algo"):
            getattr(L, name).restype = i
        _LIB = L
    return _LIB


def _check(rc):
    if rc != 0:
        raise TurboFNOError(rc, lib().turbofno_last_error_string().decode())


def _dev_c64(t, name):
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.complex64 and t.is_contiguous()):
        raise TypeError("%s must be a contiguous complex64 tensor on the GPU" % name)
    return t.data_ptr()


def _same_device(*named):
    """every tensor is a contiguous complex64 GPU tensor, all on one device (checked before any pointer is taken)"""
    dev = None
    for name, t in named:
        _dev_c64(t, name)
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise ValueError("%s is on %s, expected %s: all operands must live on one GPU" % (name, t.device, dev))


def _need(cond, fmt, *args):
    if not cond:
        raise ValueError(fmt % args)


def _numel(t, name, n):
    _need(t.numel() == n, "%s holds %d elements, the call needs exactly %d", name, t.numel(), n)


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _log2(v):
    return v.bit_length() - 1 if v > 0 and v & (v - 1) == 0 else -1


def set_1d_algo(algo):
    """Process-wide choice of the fused 1D kernel (0 = by size; see include/turbofno.h). Returns the previous value."""
    prev = lib().turbofno_get_1d_algo()
    _check(lib().turbofno_set_1d_algo(int(algo)))
    return prev


def set_exchange_wait_us(microseconds):
    """Bound of the inter-block waits of the clustered 1D kernel (include/turbofno.h); 0 = give up at once."""
    _check(lib().turbofno_set_exchange_wait_us(int(microseconds)))


def exchange_bytes(compute_units=0):
    """Size of an exchange buffer for clustered 1D launches (0 = the current device; needs a GPU then)."""
    return int(lib().turbofno_exchange_bytes(int(compute_units)))


class ExchangeBuffer:
    """A caller-owned exchange buffer attached to torch's current stream (turbofno_exchange_attach); detaches on
    close() / at the end of a `with` block. The tensor lives as long as this object."""

    def __init__(self, stream=None):
        self._stream = torch.cuda.current_stream() if stream is None else stream
        self.buffer = torch.empty(exchange_bytes(0), dtype=torch.uint8, device="cuda")
        _check(lib().turbofno_exchange_attach(self._stream.cuda_stream, self.buffer.data_ptr(), self.buffer.numel()))

    def status(self):
        """waits for the stream; number of cluster members that ran out of their wait since the last call"""
        n = ctypes.c_uint(0)
        rc = lib().turbofno_exchange_status(self._stream.cuda_stream, ctypes.byref(n))
        if rc not in (0, 5):
            _check(rc)
        return int(n.value)

    def close(self):
        if self.buffer is not None:
            _check(lib().turbofno_exchange_detach(self._stream.cuda_stream))
            self._stream.synchronize()          # enqueued work may still use the memory
            self.buffer = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
        return False


def query_2d_algo(bs, DX, DY, K, N, algo=0):
    """The algorithm layer_2d runs for these sizes (1 three kernels, 2 whole image, 3 rows first; 0 = refused)."""
    return int(lib().turbofno_query_2d_algo(bs, DX, DY, K, N, algo))


def query_1d_kernel(DY, S, N, K, compute_units=256, exchange_attached=False):
    """The fused 1D kernel (numbering of set_1d_algo, 1 ... 8) for S signals per channel; 0 = refused. With an explicit
    compute_units this is pure arithmetic (no GPU needed)."""
    return int(lib().turbofno_query_1d_kernel(_log2(DY), MODES * S, N, K, int(compute_units), 1 if exchange_attached else 0))


def fused_fft_cgemm_ifft(M, N, K, x, W, y, alpha=1.0 + 0j, beta=0j, C=None):
    """Fused 1D layer kernel: x[K][S][DY] -> y[N][S][DY], W[k + n*K], M = 64*S (reference signature
    fused_fft_cgemm_ifft_7.cuh:9; C and beta are unused there and here)."""
    DY = x.shape[-1]
    _need(M > 0 and M % MODES == 0, "M=%d must be a positive multiple of %d", M, MODES)
    S = M // MODES
    _numel(x, "x", K * S * DY)
    _numel(W, "W", K * N)
    _numel(y, "y", N * S * DY)
    _same_device(("x", x), ("W", W), ("y", y))
    a, b = complex(alpha), complex(beta)
    _check(lib().turbofno_fused_fft_cgemm_ifft(_log2(DY), M, N, K, x.data_ptr(), W.data_ptr(),
                                               None if C is None else _dev_c64(C, "C"), y.data_ptr(),
                                               a.real, a.imag, b.real, b.imag, _stream()))
    return y


def _stride_args(inp, out, DY, total, dimX, DX):
    _need(DY > 0 and total > 0 and total % DY == 0, "total=%d must be a positive multiple of DY=%d", total, DY)
    return total // DY


def fft_stride(inp, out, threadblock_bs, DY, total, dimX=MODES):
    """X-axis truncated forward transform: in[total/DY][DX][DY] -> out[total/DY][dimX][DY]."""
    DX = inp.shape[-2]
    nsig = _stride_args(inp, out, DY, total, dimX, DX)
    _numel(inp, "in", nsig * DX * DY)
    _numel(out, "out", nsig * dimX * DY)
    _same_device(("in", inp), ("out", out))
    _check(lib().turbofno_fft_stride(_log2(DX), inp.data_ptr(), out.data_ptr(), threadblock_bs, DY,
                                     total, dimX, _stream()))
    return out


def ifft_stride(inp, out, threadblock_bs, DY, total, dimX=MODES):
    """X-axis zero-padded backward transform: in[total/DY][dimX][DY] -> out[total/DY][DX][DY]."""
    DX = out.shape[-2]
    nsig = _stride_args(inp, out, DY, total, dimX, DX)
    _numel(inp, "in", nsig * dimX * DY)
    _numel(out, "out", nsig * DX * DY)
    _same_device(("in", inp), ("out", out))
    _check(lib().turbofno_ifft_stride(_log2(DX), inp.data_ptr(), out.data_ptr(), threadblock_bs, DY,
                                      total, dimX, _stream()))
    return out


def layer_1d(x, W, y=None, alpha=1.0 + 0j, dimX=1):
    """x: [K][bs*dimX][DY], W: [N][K] (element W[k + n*K]) -> y: [N][bs*dimX][DY]."""
    _need(x.dim() == 3 and W.dim() == 2, "x must be [K][S][DY] and W [N][K]")
    K, S, DY = x.shape
    N = W.shape[0]
    _need(W.shape[1] == K, "W is [%d][%d] but x has K=%d channels", W.shape[0], W.shape[1], K)
    _need(dimX > 0 and S % dimX == 0, "S=%d signals per channel is not a multiple of dimX=%d", S, dimX)
    if y is None:
        y = torch.empty((N, S, DY), dtype=torch.complex64, device=x.device)
    _need(tuple(y.shape) == (N, S, DY), "y has shape %s, expected %s", tuple(y.shape), (N, S, DY))
    _same_device(("x", x), ("W", W), ("y", y))
    a = complex(alpha)
    _check(lib().turbofno_layer_1d(S // dimX, dimX, DY, K, N, x.data_ptr(), W.data_ptr(), y.data_ptr(),
                                   a.real, a.imag, _stream()))
    return y


def layer_2d_workspace_bytes(bs, DX, DY, K, N, algo=0):
    return int(lib().turbofno_layer_2d_workspace_bytes(bs, DX, DY, K, N, algo))


def _layer_2d_operands(x, W, y):
    _need(x.dim() == 4 and W.dim() == 2, "x must be [K][bs][DX][DY] and W [N][K]")
    K, bs, DX, DY = x.shape
    N = W.shape[0]
    _need(W.shape[1] == K, "W is [%d][%d] but x has K=%d channels", W.shape[0], W.shape[1], K)
    if y is None:
        y = torch.empty((N, bs, DX, DY), dtype=torch.complex64, device=x.device)
    _need(tuple(y.shape) == (N, bs, DX, DY), "y has shape %s, expected %s", tuple(y.shape), (N, bs, DX, DY))
    _same_device(("x", x), ("W", W), ("y", y))
    return K, bs, DX, DY, N, y


def layer_2d(x, W, y=None, alpha=1.0 + 0j, workspace=None, algo=0):
    """x: [K][bs][DX][DY], W: [N][K] -> y: [N][bs][DX][DY]. `workspace`: uint8 GPU tensor (allocated
    here when omitted; pass one to keep allocation out of a timed loop). algo: 0 by size, 1 three kernels with the X
    axis first, 2 one block per image, 3 three kernels with whole rows first."""
    K, bs, DX, DY, N, y = _layer_2d_operands(x, W, y)
    need = layer_2d_workspace_bytes(bs, DX, DY, K, N, algo)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    if not (isinstance(workspace, torch.Tensor) and workspace.is_cuda and workspace.dtype == torch.uint8
            and workspace.is_contiguous()):
        raise TypeError("workspace must be a contiguous uint8 tensor on the GPU")
    _need(workspace.device == x.device, "workspace is on %s, x on %s", workspace.device, x.device)
    a = complex(alpha)
    _check(lib().turbofno_layer_2d(bs, DX, DY, K, N, x.data_ptr(), W.data_ptr(), y.data_ptr(),
                                   a.real, a.imag, workspace.data_ptr(), workspace.numel(), algo, _stream()))
    return y


def layer_2d_noalloc(x, W, y, alpha=1.0 + 0j, algo=0):
    """turbofno_layer_2d_noalloc: the 2D layer with its intermediates in the library's static device scratch.
    `y` must be passed: nothing is allocated on this path."""
    if y is None:
        raise TypeError("y must be passed: this path allocates nothing")
    K, bs, DX, DY, N, y = _layer_2d_operands(x, W, y)
    a = complex(alpha)
    _check(lib().turbofno_layer_2d_noalloc(bs, DX, DY, K, N, x.data_ptr(), W.data_ptr(), y.data_ptr(),
                                           a.real, a.imag, algo, _stream()))
    return y


def fft2d_trunc(x, spec):
    """x: [nimg][DX][DY], DX in {128, 256}, DY in {128, 256, 512, 1024} -> spec: [nimg][4096] (retained 64 x 64 modes,
    kernel-private order)."""
    _need(x.dim() >= 2, "x must end in [DX][DY]")
    nimg = x.numel() // (x.shape[-1] * x.shape[-2])
    _need(nimg > 0, "x holds no image")
    _numel(spec, "spec", nimg * MODES * MODES)
    _same_device(("x", x), ("spec", spec))
    _check(lib().turbofno_fft2d_trunc(x.shape[-2], x.shape[-1], x.data_ptr(), spec.data_ptr(), nimg, _stream()))
    return spec


def ifft2d_pad(spec, y):
    """spec: [nimg][4096] -> y: [nimg][DX][DY]."""
    _need(y.dim() >= 2, "y must end in [DX][DY]")
    nimg = y.numel() // (y.shape[-1] * y.shape[-2])
    _need(nimg > 0, "y holds no image")
    _numel(spec, "spec", nimg * MODES * MODES)
    _same_device(("spec", spec), ("y", y))
    _check(lib().turbofno_ifft2d_pad(y.shape[-2], y.shape[-1], spec.data_ptr(), y.data_ptr(), nimg, _stream()))
    return y


def cgemm(M, N, K, A, B, C, alpha=1.0 + 0j, beta=0j):
    """C[m + n*M] = alpha * sum_k A[m + k*M] B[k + n*K] + beta * C  (A: [K][M], B: [N][K], C: [N][M] as tensors)."""
    _numel(A, "A", M * K)
    _numel(B, "B", K * N)
    _numel(C, "C", M * N)
    _same_device(("A", A), ("B", B), ("C", C))
    a, b = complex(alpha), complex(beta)
    _check(lib().turbofno_cgemm(M, N, K, A.data_ptr(), B.data_ptr(), C.data_ptr(), a.real, a.imag,
                                b.real, b.imag, _stream()))
    return C


def fft_stride_DY(inp, out, threadblock_bs, total):
    """Contiguous truncated forward transform: in[total][DY] -> out[total][64]."""
    _numel(inp, "in", total * inp.shape[-1])
    _numel(out, "out", total * MODES)
    _same_device(("in", inp), ("out", out))
    _check(lib().turbofno_fft_stride_DY(_log2(inp.shape[-1]), inp.data_ptr(), out.data_ptr(),
                                        threadblock_bs, total, _stream()))
    return out


def ifft_stride_DY(inp, out, threadblock_bs, total):
    """Contiguous zero-padded backward transform: in[total][64] -> out[total][DY]."""
    _numel(inp, "in", total * MODES)
    _numel(out, "out", total * out.shape[-1])
    _same_device(("in", inp), ("out", out))
    _check(lib().turbofno_ifft_stride_DY(_log2(out.shape[-1]), inp.data_ptr(), out.data_ptr(),
                                         threadblock_bs, total, _stream()))
    return out


def fused_fft_cgemm(M, N, K, x, W, C, alpha=1.0 + 0j, beta=0j):
    """Variant B's first kernel: C[N][M] = alpha * FFT_trunc(x) W + beta C, x: [K][S][DY]."""
    _need(M > 0 and M % MODES == 0, "M=%d must be a positive multiple of %d", M, MODES)
    _numel(x, "x", K * (M // MODES) * x.shape[-1])
    _numel(W, "W", K * N)
    _numel(C, "C", M * N)
    _same_device(("x", x), ("W", W), ("C", C))
    a, b = complex(alpha), complex(beta)
    _check(lib().turbofno_fused_fft_cgemm(_log2(x.shape[-1]), M, N, K, x.data_ptr(), W.data_ptr(),
                                          C.data_ptr(), a.real, a.imag, b.real, b.imag, _stream()))
    return C


def fused_cgemm_ifft(M, N, K, A, W, y, alpha=1.0 + 0j):
    """Variant C's second kernel: y[N][S][DY] = iFFT_pad(alpha * A W), A: [K][M]."""
    _need(M > 0 and M % MODES == 0, "M=%d must be a positive multiple of %d", M, MODES)
    _numel(A, "A", M * K)
    _numel(W, "W", K * N)
    _numel(y, "y", N * (M // MODES) * y.shape[-1])
    _same_device(("A", A), ("W", W), ("y", y))
    a = complex(alpha)
    _check(lib().turbofno_fused_cgemm_ifft(_log2(y.shape[-1]), M, N, K, A.data_ptr(), W.data_ptr(), None,
                                           y.data_ptr(), a.real, a.imag, 0.0, 0.0, _stream()))
    return y
