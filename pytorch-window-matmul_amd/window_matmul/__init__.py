"""Banded ("windowed") batched matmuls for local attention on MI355X.

Drop-in for the ``window_matmul`` package of webis-de/pytorch-window-matmul
(reference window_matmul/__init__.py:1-4): same two public functions, same
autograd behaviour, with gfx950 HIP kernels underneath.
"""
from .band_softmax import BandSoftmaxFunc, band_softmax  # addition; deliberately not in __all__
from .window_attention import WindowAttentionFunc, window_attention  # addition; not in __all__
from .window_matmul import (
    UnwindowMatmulFunc,
    WindowMatmulFunc,
    unwindow_matmul,
    window_matmul,
)

__all__ = ["window_matmul", "unwindow_matmul"]
