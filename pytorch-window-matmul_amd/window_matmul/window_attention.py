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


# tensors below this many elements: the step is bound by the host's launches, of which the fused path has fewer
_HOST_BOUND_ELEMENTS = 32 << 20


def _chain_is_faster(window_size: int, width: int, elements: int) -> bool:
    """Whether a training step is faster through the separate ops than through the fused kernels.
    Up to N = 64 the fused backward is one kernel at narrow windows and the fused step wins or ties at
    every window (N = 16, 32 at w <= 2: 0.67 / 0.69 and 0.48 / 0.48 ms, chain / fused, on 100 M elements:
    a tie, left to the fused kernels).  Above N = 64 the recomputing two-kernel backward costs the same
    at every narrow window, and the chain wins up to w = 32 at N = 128 (B16 M32768: 0.374 / 0.535 ms at
    w = 4, 0.510 / 0.543 at w = 32, 0.588 / 0.580 at w = 36; B96 M4096: 0.378 / 0.395 at w = 32, 0.435 /
    0.426 at w = 36) and up to about w = 24 at N = 96 (B96 M4096: 0.251 / 0.294 at w = 16, 0.332 / 0.308 at
    w = 32).  Small problems are bound by the host, which issues seven launches for the chain and three
    for the fused step: at B7 M3001 the chain takes 0.21 ms and the fused step 0.085-0.09 ms whatever the
    window and head width, so below about 32 M elements per tensor the fused kernels are always taken."""
    if width <= 64 or elements < _HOST_BOUND_ELEMENTS:
        return False
    return window_size <= (24 if width <= 96 else 32)


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
    if _native.window_attention_supported(q, window_size, scale) and not (training and _chain_is_faster(window_size, q.shape[-1], q.numel())):
        out = WindowAttentionFunc.apply(q, k, v, window_size, scale, bool(mask_out_of_range))
    else:
        att = window_matmul(q, k.transpose(-1, -2), window_size)
        out = unwindow_matmul(band_softmax(att, scale, mask_out_of_range), v, window_size)
    return out.reshape(query.shape)
