"""Window attention as the reference's callers compose it, float64.  TEST INFRASTRUCTURE ONLY.

``o = unwindow_matmul(softmax(scale * window_matmul(q, k^T, w), -1), v, w)``
(reference tests/test_attention.py:57-63), built from the pinned pieces of this package:
the dense masked-matmul oracle for the two banded products and the numpy band softmax.
Also returns the natural-log sum of exponentials of every band row, which the fused
kernel stores for its backward.  Pinned in tests/test_oracle_attention.py against two
formulations that share no code with it: sliding-window attention over zero-padded keys
and values (the unmasked semantics) and dense attention with an additive band mask (the
masked semantics), both with torch autograd for the gradients.
"""
import numpy as np
import torch

from . import dense_oracle, softmax_oracle


def window_attention_forward(q, k, v, w, scale=1.0, mask_out_of_range=False):
    """q, k, v torch tensors (B, M, N), k holding key rows.  Returns (o, lse) as float64 numpy."""
    band = dense_oracle.dense_window_matmul(q, k.transpose(1, 2), w).numpy()  # float64, +0 where invalid
    probs = softmax_oracle.band_softmax_forward(band, scale, mask_out_of_range)
    o = dense_oracle.dense_unwindow_matmul(torch.from_numpy(probs), v, w).numpy()
    M = q.shape[1]
    x = band * float(scale)
    if mask_out_of_range:
        x = np.where(softmax_oracle.valid_mask(M, w)[None], x, -np.inf)
    top = x.max(-1, keepdims=True)
    lse = (top + np.log(np.exp(x - top).sum(-1, keepdims=True)))[..., 0]
    return o, lse


def window_attention_backward(q, k, v, w, grad_o, scale=1.0, mask_out_of_range=False):
    """Gradients (dq, dk, dv) of the chain above, float64 numpy, through the pinned backward pieces."""
    kt = k.transpose(1, 2)
    band = dense_oracle.dense_window_matmul(q, kt, w).numpy()
    probs = softmax_oracle.band_softmax_forward(band, scale, mask_out_of_range)
    dprobs, dv = dense_oracle.dense_unwindow_matmul_backward(torch.from_numpy(probs), v, w, grad_o)
    dband = softmax_oracle.band_softmax_backward(probs, dprobs.numpy(), scale, mask_out_of_range)
    dq, dkt = dense_oracle.dense_window_matmul_backward(q, kt, w, torch.from_numpy(dband))
    return dq.numpy(), dkt.transpose(1, 2).numpy(), dv.numpy()
