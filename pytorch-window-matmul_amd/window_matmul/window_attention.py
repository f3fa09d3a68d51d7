"""Window attention in one call: ``unwindow_matmul(softmax(scale * window_matmul(q, k^T, w)), v, w)``.

The reference package stops at the two banded matmuls; its callers write the chain above
themselves (reference tests/test_attention.py:57-63).  This function is that chain with the
same semantics, as an addition next to the unchanged two-function API.  For float16 /
bfloat16 inputs whose last dimension is a multiple of 16 up to 128 it runs fused kernels that
never write the ``(…, M, 2w+1)`` band to memory (forward keeps only the log-sum-exp of every
row, backward recomputes the probabilities); everything else runs the chain of the separate
ops of this package, on the GPU as well.
"""
import math
from typing import Optional

import torch

import window_matmul_kernel as _native

from .band_softmax import band_softmax
from .window_matmul import unwindow_matmul, window_matmul


def _chain_is_faster(window_size: int, width: int) -> bool:
    """Windows at which a training step is faster through the separate ops than through the fused
    kernels.  Up to N = 64 the fused backward is one kernel at windows up to 32 and the chain only wins
    at the very narrowest windows of the narrow heads; above N = 64 the recomputing two-kernel backward
    costs the same at every narrow window.  Measured on bf16 tensors of 100 M elements with M = 16384
    (chain / fused, ms per step): N = 16: 0.67 / 0.69 at w = 2, 0.72 / 0.72 at w = 3; N = 32: 0.48 /
    0.48 at w = 2, 0.50 / 0.48 at w = 3; N = 48: 0.51 / 0.46 at w = 1; N = 64: 0.47 / 0.47 at w = 1,
    0.48 / 0.45 at w = 2, 0.52 / 0.44 at w = 8, 0.88 / 0.52 at w = 32; N = 96: 0.81 / 0.86 at w = 32,
    0.96 / 0.92 at w = 40; N = 128: 0.72 / 0.79 at w = 32, 0.86 / 0.84 at w = 40."""
    return window_size <= (2 if width <= 32 else 0 if width <= 64 else 36)


class WindowAttentionFunc(torch.autograd.Function):
    """Fused kernels on 3-D ``(B, M, N)`` operands; ``k`` holds key rows (not transposed)."""

    @staticmethod
    def forward(ctx, q, k, v, window_size: int, scale: float, mask_out_of_range: bool):
        out, lse = _native.window_attention_forward(q, k, v, window_size, scale, mask_out_of_range)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.window_size = window_size
        ctx.scale = scale
        return out

    @staticmethod
    def backward(ctx, grad_output):
        q, k, v, out, lse = ctx.saved_tensors
        gq, gk, gv = _native.window_attention_backward(q, k, v, out, lse, grad_output, ctx.window_size, ctx.scale,
                                                       *ctx.needs_input_grad[:3])
        return gq, gk, gv, None, None, None


def window_attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, window_size: int,
                     scale: Optional[float] = None, mask_out_of_range: bool = False) -> torch.Tensor:
    """Local attention of every position over its ``2 * window_size + 1`` neighbours.

    ``query``, ``key``, ``value`` are ``(..., M, N)`` (``key`` NOT transposed, unlike the second
    argument of ``window_matmul``); the result is ``(..., M, N)``.  ``scale`` defaults to
    ``1 / sqrt(N)``.  With ``mask_out_of_range=False`` (default) the result equals the reference
    callers' chain exactly as they write it: neighbours that fall outside the sequence take part
    in the softmax with score 0 and add nothing to the output.  With ``True`` they are left out
    of the softmax, which is the usual definition of sliding-window attention.
    """
    if query.shape != key.shape or query.shape != value.shape or query.dim() < 2:
        raise RuntimeError("Input mismatch")
    scale = 1.0 / math.sqrt(query.shape[-1]) if scale is None else float(scale)
    if not window_size:
        # a single neighbour: the softmax is 1 and the output is the value itself, as in the
        # chain (reference tests/test_attention.py:75-87); kept differentiable through torch ops
        score = (query * key).sum(-1, keepdim=True) * scale
        return torch.softmax(score, -1) * value
    q, k, v = (t.reshape(-1, t.shape[-2], t.shape[-1]) for t in (query, key, value))
    # With a very narrow band the recomputing backward of the fused kernels costs more than the
    # band it avoids writing, so training there goes through the separate ops.
    training = torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v))
    if _native.window_attention_supported(q, window_size, scale) and not (training and _chain_is_faster(window_size, q.shape[-1])):
        out = WindowAttentionFunc.apply(q, k, v, window_size, scale, bool(mask_out_of_range))
    else:
        att = window_matmul(q, k.transpose(-1, -2), window_size)
        out = unwindow_matmul(band_softmax(att, scale, mask_out_of_range), v, window_size)
    return out.reshape(query.shape)
