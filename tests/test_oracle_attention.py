"""Pins oracle/attention_oracle.py on the CPU against formulations that share no code with it."""
import math

import numpy as np
import pytest
import torch

from oracle import attention_oracle as ao
from conftest import seeded

CASES = [(2, 1, 4, 1), (2, 9, 4, 2), (1, 20, 8, 4), (3, 12, 5, 16), (2, 40, 8, 7)]  # (B, M, N, w)


def padded_sliding_attention(q, k, v, w, scale):
    """Unmasked semantics: every query sees exactly 2w+1 keys of a sequence padded with w zero
    rows on both sides; a zero key scores 0 and a zero value adds nothing."""
    B, M, N = q.shape
    zeros = torch.zeros(B, w, N, dtype=q.dtype)
    kp, vp = torch.cat([zeros, k, zeros], 1), torch.cat([zeros, v, zeros], 1)
    idx = torch.arange(M).unsqueeze(1) + torch.arange(2 * w + 1).unsqueeze(0)  # (M, 2w+1) into the padded axis
    scores = torch.einsum("bmn,bmjn->bmj", q, kp[:, idx]) * scale
    probs = torch.softmax(scores, -1)
    return torch.einsum("bmj,bmjn->bmn", probs, vp[:, idx]), torch.logsumexp(scores, -1)


def dense_band_attention(q, k, v, w, scale):
    """Masked semantics: dense attention with minus infinity outside |i - c| <= w."""
    M = q.shape[1]
    i = torch.arange(M)
    allowed = (i.unsqueeze(1) - i.unsqueeze(0)).abs() <= w
    scores = (torch.bmm(q, k.transpose(1, 2)) * scale).masked_fill(~allowed, float("-inf"))
    return torch.bmm(torch.softmax(scores, -1), v), torch.logsumexp(scores, -1)


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%d_M%d_N%d_w%d" % c)
@pytest.mark.parametrize("masked", [False, True], ids=["zero_filled", "masked"])
def test_forward_and_gradients(case, masked):
    B, M, N, w = case
    scale = 1.0 / math.sqrt(N)
    q0, k0, v0, go = (seeded((B, M, N), s, torch.float64) for s in (41, 42, 43, 44))
    q, k, v = (t.clone().requires_grad_(True) for t in (q0, k0, v0))
    want_o, want_lse = (dense_band_attention if masked else padded_sliding_attention)(q, k, v, w, scale)
    want_o.backward(go)
    o, lse = ao.window_attention_forward(q0, k0, v0, w, scale, masked)
    np.testing.assert_allclose(o, want_o.detach().numpy(), rtol=1e-11, atol=1e-13)
    np.testing.assert_allclose(lse, want_lse.detach().numpy(), rtol=1e-11, atol=1e-13)
    dq, dk, dv = ao.window_attention_backward(q0, k0, v0, w, go, scale, masked)
    for got, want in ((dq, q.grad), (dk, k.grad), (dv, v.grad)):
        np.testing.assert_allclose(got, want.numpy(), rtol=1e-10, atol=1e-12)
