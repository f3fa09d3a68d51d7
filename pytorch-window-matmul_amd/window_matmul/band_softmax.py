"""Softmax over the band dimension, the step between ``window_matmul`` and ``unwindow_matmul``.

The reference package has no such function: its callers write
``softmax(att / sqrt(N), dim=-1)`` with torch between the two ops
(reference tests/test_attention.py:60-61).  Band rows have odd length ``2w+1``, which
torch's generic softmax handles poorly; this one streams the band through LDS in
aligned 16-byte pieces.  It is an addition next to the unchanged two-function API, not
part of ``window_matmul.__all__``.
"""
from typing import Optional

import torch

import window_matmul_kernel as _native


class BandSoftmaxFunc(torch.autograd.Function):
    """``softmax(scale * inp, dim=-1)`` on a 3-D band ``(B, M, 2w+1)``; saves only the result."""

    @staticmethod
    def forward(ctx, inp: torch.Tensor, scale: float, mask_out_of_range: bool) -> torch.Tensor:
        probs = _native.band_softmax_forward(inp, scale, mask_out_of_range)
        ctx.save_for_backward(probs)
        ctx.scale = scale
        ctx.mask_out_of_range = mask_out_of_range
        return probs

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        (probs,) = ctx.saved_tensors
        return _native.band_softmax_backward(probs, grad_output, ctx.scale, ctx.mask_out_of_range), None, None


def band_softmax(inp: torch.Tensor, scale: Optional[float] = None, mask_out_of_range: bool = False) -> torch.Tensor:
    """``softmax(scale * inp, dim=-1)`` for a band tensor ``(..., M, 2w+1)``.

    With ``mask_out_of_range=False`` (default) the result equals
    ``torch.softmax(inp * scale, -1)``: the entries of a row that refer to positions outside
    the sequence take part with whatever they hold (``window_matmul`` leaves ``0.0`` there),
    which is what callers of the reference get.  With ``mask_out_of_range=True`` those
    entries are treated as ``-inf``: probability and gradient exactly ``0.0``.
    Computes in float32 (float64 for double tensors) and returns the input's dtype.
    """
    if inp.dim() < 2 or inp.shape[-1] % 2 != 1:
        raise RuntimeError("Input mismatch")
    scale = 1.0 if scale is None else float(scale)
    flat = inp.reshape(-1, inp.shape[-2], inp.shape[-1])
    return BandSoftmaxFunc.apply(flat, scale, bool(mask_out_of_range)).reshape(inp.shape)
