"""Pins oracle/softmax_oracle.py without a GPU: against torch.softmax and its autograd on the
CPU (what the reference's callers run, reference tests/test_attention.py:60-61) and against
closed forms that a wrong mask, a dropped scale or a wrong sign would break."""
import numpy as np
import pytest
import torch

from oracle import softmax_oracle as so
from conftest import seeded


@pytest.mark.parametrize("B,M,w", [(2, 1, 0), (2, 7, 1), (1, 20, 4), (3, 9, 16), (2, 50, 33)])
@pytest.mark.parametrize("scale", [1.0, 0.125, -0.7])
def test_matches_torch_softmax_and_autograd(B, M, w, scale):
    a = seeded((B, M, 2 * w + 1), 5, torch.float64)
    g = seeded((B, M, 2 * w + 1), 6, torch.float64)
    x = a.clone().requires_grad_(True)
    p = torch.softmax(x * scale, -1)
    p.backward(g)
    got_p = so.band_softmax_forward(a.numpy(), scale)
    np.testing.assert_allclose(got_p, p.detach().numpy(), rtol=1e-12, atol=1e-15)
    got_g = so.band_softmax_backward(got_p, g.numpy(), scale)
    np.testing.assert_allclose(got_g, x.grad.numpy(), rtol=1e-10, atol=1e-14)


@pytest.mark.parametrize("B,M,w", [(2, 7, 1), (1, 20, 4), (3, 9, 16), (2, 50, 33)])
def test_masked_matches_torch_with_minus_infinity(B, M, w):
    a = seeded((B, M, 2 * w + 1), 7, torch.float64)
    g = seeded((B, M, 2 * w + 1), 8, torch.float64)
    keep = torch.from_numpy(so.valid_mask(M, w))
    x = a.clone().requires_grad_(True)
    p = torch.softmax((x * 0.5).masked_fill(~keep, float("-inf")), -1)
    p.backward(g)
    got_p = so.band_softmax_forward(a.numpy(), 0.5, True)
    np.testing.assert_allclose(got_p, p.detach().numpy(), rtol=1e-12, atol=1e-15)
    assert (got_p[:, ~keep.numpy()] == 0).all()
    got_g = so.band_softmax_backward(got_p, g.numpy(), 0.5, True)
    np.testing.assert_allclose(got_g, x.grad.numpy(), rtol=1e-10, atol=1e-14)
    # garbage in masked entries of the inputs changes nothing
    a2 = a.numpy().copy()
    a2[:, ~keep.numpy()] = np.nan
    g2 = g.numpy().copy()
    g2[:, ~keep.numpy()] = np.inf
    np.testing.assert_array_equal(so.band_softmax_forward(a2, 0.5, True), got_p)
    np.testing.assert_array_equal(so.band_softmax_backward(got_p, g2, 0.5, True), got_g)


def test_closed_forms():
    M, w = 12, 3
    W = 2 * w + 1
    ones = np.ones((1, M, W))
    # uniform rows: 1/W unmasked, 1/(number of in-sequence entries) masked
    np.testing.assert_allclose(so.band_softmax_forward(ones, 3.0), 1.0 / W)
    counts = so.valid_mask(M, w).sum(-1)
    assert counts.tolist() == [min(M - 1, i + w) - max(0, i - w) + 1 for i in range(M)]
    pm = so.band_softmax_forward(ones, 3.0, True)
    np.testing.assert_allclose(pm.sum(-1), 1.0)
    np.testing.assert_allclose(pm.max(-1)[0], 1.0 / counts)
    # two-entry row: logistic function of the scaled difference
    a = np.zeros((1, 1, 1)) + 0.0
    assert so.band_softmax_forward(a).item() == 1.0
    a = np.array([[[0.0, 2.0, -1e9]]])  # w = 1, M = 1 -> only the centre is in sequence
    np.testing.assert_allclose(so.band_softmax_forward(a, 0.5)[0, 0, :2], [1 / (1 + np.e), np.e / (1 + np.e)])
    assert so.band_softmax_forward(a, 0.5, True)[0, 0].tolist() == [0.0, 1.0, 0.0]
    # shift invariance and gradient rows summing to zero
    x = np.random.default_rng(0).normal(size=(2, M, W))
    p = so.band_softmax_forward(x, 0.3)
    np.testing.assert_allclose(so.band_softmax_forward(x + 5.0, 0.3), p, rtol=1e-12)
    g = so.band_softmax_backward(p, np.random.default_rng(1).normal(size=p.shape), 0.3)
    np.testing.assert_allclose(g.sum(-1), 0.0, atol=1e-15)
