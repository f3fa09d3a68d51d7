"""Softmax over the band dimension, float64 numpy.  TEST INFRASTRUCTURE ONLY.

Restates what the reference's callers compute with torch between the two ops
(reference tests/test_attention.py:60-61): ``softmax(scale * a, dim=-1)`` over all
``2w+1`` entries of a band row.  With ``mask_out_of_range`` the entries whose source
position ``i + j - w`` lies outside ``[0, M)`` (reference tests/utils.py:79-81) count
as minus infinity.  Pinned in tests/test_oracle_softmax.py against ``torch.softmax``
and its autograd on the CPU and against closed forms.
"""
import numpy as np


def valid_mask(M: int, w: int) -> np.ndarray:
    i = np.arange(M)[:, None]
    j = np.arange(2 * w + 1)[None, :]
    c = i + j - w
    return (c >= 0) & (c < M)


def band_softmax_forward(a: np.ndarray, scale: float = 1.0, mask_out_of_range: bool = False) -> np.ndarray:
    """a (B, M, 2w+1) -> probabilities, float64."""
    B, M, W = a.shape
    x = a.astype(np.float64) * float(scale)
    keep = valid_mask(M, W // 2) if mask_out_of_range else np.ones((M, W), dtype=bool)
    x = np.where(keep[None], x, -np.inf)
    top = x.max(axis=-1, keepdims=True)
    e = np.where(keep[None], np.exp(x - top), 0.0)
    return e / e.sum(axis=-1, keepdims=True)


def band_softmax_backward(p: np.ndarray, grad_p: np.ndarray, scale: float = 1.0,
                          mask_out_of_range: bool = False) -> np.ndarray:
    """grad wrt a from saved probabilities: scale * p * (g - sum_j p_j g_j); masked entries +0."""
    B, M, W = p.shape
    keep = valid_mask(M, W // 2) if mask_out_of_range else np.ones((M, W), dtype=bool)
    pp = np.where(keep[None], p.astype(np.float64), 0.0)
    gg = np.where(keep[None], grad_p.astype(np.float64), 0.0)
    dot = (pp * gg).sum(axis=-1, keepdims=True)
    return np.where(keep[None], float(scale) * pp * (gg - dot), 0.0)
