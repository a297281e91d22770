"""CPU-only checks of the Python binding's operand validation: mismatched shapes are refused before any pointer
reaches the C ABI (a wrong size there would be an out-of-bounds device access), and correctly shaped operands that
are not GPU tensors are refused as such. No GPU call is made."""
import pytest
import torch

import turbofno_amd as tf


def c64(*shape):
    return torch.zeros(shape, dtype=torch.complex64)


def test_layer_1d_rejects_mismatched_operands():
    x, W = c64(8, 6, 128), c64(64, 8)
    with pytest.raises(ValueError, match="K=8"):
        tf.layer_1d(x, c64(64, 16))                       # W's K differs from x's
    with pytest.raises(ValueError, match="dimX"):
        tf.layer_1d(x, W, dimX=4)                         # 6 signals are not a multiple of dimX = 4
    with pytest.raises(ValueError, match="y has shape"):
        tf.layer_1d(x, W, y=c64(64, 5, 128))
    with pytest.raises(ValueError):
        tf.layer_1d(c64(8, 128), W)                       # x is not [K][S][DY]
    with pytest.raises(TypeError, match="on the GPU"):
        tf.layer_1d(x, W, y=c64(64, 6, 128))              # consistent shapes, but host tensors


def test_layer_2d_rejects_mismatched_operands():
    x, W = c64(8, 1, 128, 128), c64(64, 8)
    with pytest.raises(ValueError, match="K=8"):
        tf.layer_2d(x, c64(64, 24))
    with pytest.raises(ValueError, match="y has shape"):
        tf.layer_2d(x, W, y=c64(64, 1, 128, 256))
    with pytest.raises(ValueError, match="y has shape"):
        tf.layer_2d_noalloc(x, W, c64(64, 2, 128, 128))
    with pytest.raises(TypeError):
        tf.layer_2d_noalloc(x, W, None)
    with pytest.raises(TypeError, match="on the GPU"):
        tf.layer_2d(x, W, y=c64(64, 1, 128, 128))


def test_kernel_table_entry_points_reject_wrong_sizes():
    x, W, y = c64(8, 2, 128), c64(64, 8), c64(64, 2, 128)
    with pytest.raises(ValueError, match="multiple of 64"):
        tf.fused_fft_cgemm_ifft(100, 64, 8, x, W, y)
    with pytest.raises(ValueError, match="x holds"):
        tf.fused_fft_cgemm_ifft(64 * 3, 64, 8, x, W, y)   # M says three signals, x has two
    with pytest.raises(ValueError, match="y holds"):
        tf.fused_fft_cgemm_ifft(64 * 2, 128, 8, x, c64(128, 8), y)
    with pytest.raises(ValueError, match="W holds"):
        tf.fused_fft_cgemm_ifft(64 * 2, 64, 8, x, c64(64, 16), y)
    with pytest.raises(TypeError, match="on the GPU"):
        tf.fused_fft_cgemm_ifft(64 * 2, 64, 8, x, W, y)


def test_stage_entry_points_reject_wrong_sizes():
    with pytest.raises(ValueError, match="multiple of DY"):
        tf.fft_stride(c64(2, 128, 32), c64(2, 64, 32), 4, 32, 70)
    with pytest.raises(ValueError, match="in holds"):
        tf.fft_stride(c64(2, 128, 32), c64(3, 64, 32), 4, 32, 96)        # total says three signals
    with pytest.raises(ValueError, match="out holds"):
        tf.ifft_stride(c64(2, 64, 32), c64(2, 128, 16), 4, 32, 64)
    with pytest.raises(ValueError, match="A holds"):
        tf.cgemm(128, 64, 8, c64(8, 64), c64(64, 8), c64(64, 128))
    with pytest.raises(ValueError, match="C holds"):
        tf.cgemm(128, 64, 8, c64(8, 128), c64(64, 8), c64(64, 64))
    with pytest.raises(ValueError, match="spec holds"):
        tf.fft2d_trunc(c64(3, 128, 128), c64(2, 4096))
    with pytest.raises(ValueError, match="spec holds"):
        tf.ifft2d_pad(c64(2, 4096), c64(3, 128, 128))
    with pytest.raises(ValueError, match="in holds"):
        tf.fft_stride_DY(c64(5, 128), c64(6, 64), 4, 6)
    with pytest.raises(ValueError, match="out holds"):
        tf.ifft_stride_DY(c64(6, 64), c64(5, 256), 4, 6)
    with pytest.raises(ValueError, match="C holds"):
        tf.fused_fft_cgemm(128, 64, 8, c64(8, 2, 128), c64(64, 8), c64(64, 64))
    with pytest.raises(ValueError, match="y holds"):
        tf.fused_cgemm_ifft(128, 64, 8, c64(8, 128), c64(64, 8), c64(64, 3, 128))
    with pytest.raises(TypeError, match="on the GPU"):
        tf.cgemm(128, 64, 8, c64(8, 128), c64(64, 8), c64(64, 128))


def test_1d_kernel_selector_round_trip():
    prev = tf.set_1d_algo(5)
    assert tf.lib().turbofno_get_1d_algo() == 5
    with pytest.raises(tf.TurboFNOError):
        tf.set_1d_algo(9)
    assert tf.lib().turbofno_get_1d_algo() == 5           # a refused value changes nothing
    tf.set_1d_algo(prev)


def test_noalloc_refuses_oversized_problem_without_gpu():
    L = tf.lib()
    # bs=32, 256 x 256, K=N=64: 128 MiB of intermediates, the static scratch holds 64 MiB; refused before any GPU call
    rc = L.turbofno_layer_2d_noalloc(32, 256, 256, 64, 64, 1, 1, 1, 1.0, 0.0, 2, None)
    assert rc == 3 and b"static scratch" in L.turbofno_last_error_string()
