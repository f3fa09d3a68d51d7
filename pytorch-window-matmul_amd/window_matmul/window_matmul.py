"""Python API and autograd glue of the banded matmuls.

Mirrors reference window_matmul/window_matmul.py:7-76: the public functions
``window_matmul(inp, other, window_size)`` and ``unwindow_matmul(inp, other,
window_size)`` plus the two ``torch.autograd.Function`` classes they apply.
All arithmetic happens in the native module ``window_matmul_kernel`` (HIP
kernels for gfx950); if that module has not been built the import below fails,
on purpose -- there is no Python or CPU fallback behind this package.

Band convention: with ``W = 2 * window_size + 1``, column ``j`` of band row
``i`` refers to sequence position ``i + j - window_size``; positions outside
``[0, M)`` read as nothing and are written as exact zeros.
"""
from typing import Optional, Tuple

import torch

import window_matmul_kernel as _native

# Inside a CUDA/HIP autocast region the operands are cast to float16 and the
# body runs with autocast disabled (reference window_matmul.py:9,18,45,54).
_amp_forward = torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.float16)
_amp_backward = torch.amp.custom_bwd(device_type="cuda")


class WindowMatmulFunc(torch.autograd.Function):
    """``A[b, i, j] = sum_h inp[b, i, h] * other[b, h, i + j - w]`` on 3-D operands.

    ``inp`` is ``(B, M, N)``, ``other`` is ``(B, N, M)`` (the keys, transposed),
    the result is ``(B, M, 2w+1)``.  reference window_matmul.py:7-27.
    """

    @staticmethod
    @_amp_forward
    def forward(ctx, inp: torch.Tensor, other: torch.Tensor, window_size: int) -> torch.Tensor:
        ctx.save_for_backward(inp, other)
        return _native.window_matmul_forward(inp, other, window_size)

    @staticmethod
    @_amp_backward
    def backward(ctx, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, None]:
        inp, other = ctx.saved_tensors
        # the band width fixes the window: W = 2w + 1  (reference window_matmul.py:22)
        half_width = grad_output.shape[-1] // 2
        # a gradient nobody asked for is not computed (the reference always computes both)
        grad_inp, grad_other = _native.window_matmul_backward(
            inp, other, half_width, grad_output, ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        )
        return grad_inp, grad_other, None


class UnwindowMatmulFunc(torch.autograd.Function):
    """``O[b, i, h] = sum_j inp[b, i, j] * other[b, i + j - w, h]`` on 3-D operands.

    ``inp`` is the band ``(B, M, 2w+1)``, ``other`` is ``(B, M, N)``, the result is
    ``(B, M, N)``.  reference window_matmul.py:43-63.
    """

    @staticmethod
    @_amp_forward
    def forward(ctx, inp: torch.Tensor, other: torch.Tensor, window_size: int) -> torch.Tensor:
        ctx.save_for_backward(inp, other)
        return _native.unwindow_matmul_forward(inp, other, window_size)

    @staticmethod
    @_amp_backward
    def backward(ctx, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, None]:
        inp, other = ctx.saved_tensors
        half_width = inp.shape[-1] // 2  # reference window_matmul.py:59
        grad_inp, grad_other = _native.unwindow_matmul_backward(
            inp, other, half_width, grad_output, ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        )
        return grad_inp, grad_other, None


def window_matmul(inp: torch.Tensor, other: torch.Tensor, window_size: Optional[int]) -> torch.Tensor:
    """Band of ``inp @ other``: ``(..., M, N) x (..., N, M) -> (..., M, 2w+1)``.

    A falsy ``window_size`` keeps only the diagonal and is computed with plain
    torch ops, giving ``(..., M, 1)`` (reference window_matmul.py:33-34).  Any
    number of leading dimensions is flattened into one batch dimension for the
    kernel and restored afterwards (reference window_matmul.py:35-40).
    """
    if not window_size:
        return (inp * other.transpose(-1, -2)).sum(dim=-1, keepdim=True)
    lead = inp.shape[:-2]
    seq_len, hidden_dim = inp.shape[-2:]
    band = WindowMatmulFunc.apply(
        inp.reshape(-1, seq_len, hidden_dim), other.reshape(-1, hidden_dim, seq_len), window_size
    )
    return band.reshape(*lead, seq_len, 2 * window_size + 1)


def unwindow_matmul(inp: torch.Tensor, other: torch.Tensor, window_size: Optional[int]) -> torch.Tensor:
    """Band times values: ``(..., M, 2w+1) x (..., M, N) -> (..., M, N)``.

    A falsy ``window_size`` is the elementwise product ``inp * other``
    (reference window_matmul.py:69-70); leading dimensions are flattened and
    restored as in :func:`window_matmul` (reference window_matmul.py:71-76).
    """
    if not window_size:
        return inp * other
    lead = other.shape[:-2]
    seq_len, hidden_dim = other.shape[-2:]
    out = UnwindowMatmulFunc.apply(
        inp.reshape(-1, seq_len, 2 * window_size + 1), other.reshape(-1, seq_len, hidden_dim), window_size
    )
    return out.reshape(*lead, seq_len, hidden_dim)
