"""Dense masked-matmul statement of the banded products.  TEST INFRASTRUCTURE ONLY.

A different formulation from the loop restatement, built from library routines:
the whole ``M x M`` score matrix is formed with ``bmm`` and the band is gathered
out of it (window op), or the band is scattered into a dense ``M x M`` matrix
and multiplied with ``bmm`` (unwindow op).  Backward passes are written out as
the matching dense products.  Works on any device torch supports, in the
precision of ``work_dtype`` (float64 by default).

Band convention (reference README.md:5,9; tests/utils.py:79-81): band column
``j`` of row ``i`` addresses source row ``c = i + j - w``; it is valid iff
``0 <= c < M``.  Invalid entries of an output band are +0.0; invalid entries of
an input band are ignored whatever they hold.
"""
import torch


def band_index(M: int, w: int, device=None):
    """(c, valid): c[i, j] = i + j - w clamped into range, valid[i, j] = 0 <= i+j-w < M."""
    i = torch.arange(M, device=device).unsqueeze(1)
    j = torch.arange(2 * w + 1, device=device).unsqueeze(0)
    c = i + j - w
    valid = (c >= 0) & (c < M)
    return c.clamp(0, M - 1), valid


def band_mask(M: int, w: int, device=None) -> torch.Tensor:
    """Boolean (M, 2w+1) mask of in-sequence band entries."""
    return band_index(M, w, device)[1]


def dense_to_band(S: torch.Tensor, w: int) -> torch.Tensor:
    """(B, M, M) -> (B, M, 2w+1): band[b,i,j] = S[b,i,i+j-w], +0 where invalid."""
    M = S.shape[-1]
    c, valid = band_index(M, w, S.device)
    band = torch.gather(S, 2, c.unsqueeze(0).expand(S.shape[0], -1, -1))
    return torch.where(valid.unsqueeze(0), band, torch.zeros((), dtype=S.dtype, device=S.device))


def band_to_dense(A: torch.Tensor, w: int) -> torch.Tensor:
    """(B, M, 2w+1) -> (B, M, M): D[b,i,i+j-w] = A[b,i,j] on valid entries, 0 elsewhere.

    Invalid band entries are dropped before the scatter, so NaN/Inf planted in
    them never reaches the result."""
    B, M, _ = A.shape
    c, valid = band_index(M, w, A.device)
    clean = torch.where(valid.unsqueeze(0), A, torch.zeros((), dtype=A.dtype, device=A.device))
    D = torch.zeros(B, M, M, dtype=A.dtype, device=A.device)
    # clamped duplicates only ever add the zeros written above
    D.scatter_add_(2, c.unsqueeze(0).expand(B, -1, -1), clean)
    return D


def dense_window_matmul(q, kt, w, work_dtype=torch.float64):
    """q (B,M,N), kt (B,N,M) -> band (B,M,2w+1) in work_dtype."""
    S = torch.bmm(q.to(work_dtype), kt.to(work_dtype))
    return dense_to_band(S, w)


def dense_unwindow_matmul(a, v, w, work_dtype=torch.float64):
    """a (B,M,2w+1), v (B,M,N) -> (B,M,N) in work_dtype."""
    return torch.bmm(band_to_dense(a.to(work_dtype), w), v.to(work_dtype))


def dense_window_matmul_backward(q, kt, w, grad_a, work_dtype=torch.float64):
    """Returns (dQ (B,M,N), dK^T (B,N,M)).  dS is the upstream band scattered to dense."""
    dS = band_to_dense(grad_a.to(work_dtype), w)
    dq = torch.bmm(dS, kt.to(work_dtype).transpose(1, 2))
    dkt = torch.bmm(q.to(work_dtype).transpose(1, 2), dS)
    return dq, dkt


def dense_unwindow_matmul_backward(a, v, w, grad_o, work_dtype=torch.float64):
    """Returns (dA (B,M,2w+1), dV (B,M,N))."""
    g = grad_o.to(work_dtype)
    da = dense_to_band(torch.bmm(g, v.to(work_dtype).transpose(1, 2)), w)
    dv = torch.bmm(band_to_dense(a.to(work_dtype), w).transpose(1, 2), g)
    return da, dv
