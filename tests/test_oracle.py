"""Pins the CPU oracle before anything is compared against it.

Each check is chosen so that a plausible slip in the restatement (wrong sign in
the band index, transposed operand, dropped bound, flipped band in the
transposed products) fails at least one of them:

* bit-exact agreement with the reference's own compiled CPU path (oracle/_ref),
  where that build exists, on the reference's test grid (reference
  tests/conftest.py:5-13) and on ragged shapes;
* agreement with a dense masked matmul in float64 (a different formulation);
* closed forms: all-ones inputs, one-hot rows, sliding-window sums by cumsum;
* brute force from the README definition on tiny sizes;
* adjoint identities tying each backward to its forward;
* exact +0.0 in out-of-sequence band entries, and input-band garbage ignored.
"""
import itertools

import pytest
import torch

import oracle
from conftest import seeded

REF_DIMS = [(2, 1, 3), (2, 4, 3), (2, 16, 3), (2, 32, 3), (2, 16, 32)]  # (B, M, N)
REF_WINDOWS = [1, 4, 16]
RAGGED = [(3, 37, 5, 6), (1, 1, 7, 3), (2, 9, 8, 4), (2, 50, 16, 49), (2, 50, 16, 80), (1, 64, 24, 8)]


def _inputs(B, M, N, w, dtype=torch.float32, seed=0):
    q = seeded((B, M, N), seed, dtype)
    kt = seeded((B, M, N), seed + 1, dtype).transpose(1, 2).contiguous()
    v = seeded((B, M, N), seed + 2, dtype)
    a = seeded((B, M, 2 * w + 1), seed + 3, dtype)
    ga = seeded((B, M, 2 * w + 1), seed + 4, dtype)
    go = seeded((B, M, N), seed + 5, dtype)
    return q, kt, v, a, ga, go


def _all_cases():
    cases = [(B, M, N, w) for (B, M, N), w in itertools.product(REF_DIMS, REF_WINDOWS)]
    return cases + RAGGED


@pytest.mark.parametrize("B,M,N,w", _all_cases())
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_restatement_bit_exact_vs_compiled_reference(B, M, N, w, dtype):
    ref = oracle.reference_module()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference sources absent on this machine)")
    q, kt, v, a, ga, go = _inputs(B, M, N, w, dtype)
    assert torch.equal(oracle.window_matmul_forward(q, kt, w), ref.window_matmul_forward(q, kt, w))
    assert torch.equal(oracle.unwindow_matmul_forward(a, v, w), ref.unwindow_matmul_forward(a, v, w))
    for mine, theirs in zip(oracle.window_matmul_backward(q, kt, w, ga), ref.window_matmul_backward(q, kt, w, ga)):
        assert torch.equal(mine, theirs)
    for mine, theirs in zip(oracle.unwindow_matmul_backward(a, v, w, go), ref.unwindow_matmul_backward(a, v, w, go)):
        assert torch.equal(mine, theirs)


@pytest.mark.parametrize("B,M,N,w", _all_cases())
def test_restatement_vs_dense_masked_matmul(B, M, N, w):
    q, kt, v, a, ga, go = _inputs(B, M, N, w, torch.float64)
    tol = dict(rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(oracle.window_matmul_forward(q, kt, w), oracle.dense_window_matmul(q, kt, w), **tol)
    torch.testing.assert_close(oracle.unwindow_matmul_forward(a, v, w), oracle.dense_unwindow_matmul(a, v, w), **tol)
    dq, dkt = oracle.window_matmul_backward(q, kt, w, ga)
    rq, rkt = oracle.dense_window_matmul_backward(q, kt, w, ga)
    torch.testing.assert_close(dq, rq, **tol)
    torch.testing.assert_close(dkt, rkt, **tol)
    da, dv = oracle.unwindow_matmul_backward(a, v, w, go)
    ra, rv = oracle.dense_unwindow_matmul_backward(a, v, w, go)
    torch.testing.assert_close(da, ra, **tol)
    torch.testing.assert_close(dv, rv, **tol)


def _readme_window(q, kt, w):
    """A[i,j] = sum_h q[i,h] * k[h, i+j-w], zero out of range (reference README.md:5)."""
    B, M, N = q.shape
    out = torch.zeros(B, M, 2 * w + 1, dtype=q.dtype)
    for b, i, j in itertools.product(range(B), range(M), range(2 * w + 1)):
        c = i + j - w
        if 0 <= c < M:
            out[b, i, j] = sum(q[b, i, h] * kt[b, h, c] for h in range(N))
    return out


def _readme_unwindow(a, v, w):
    """O[i,h] = sum_j a[i,j] * v[i+j-w, h] over in-range j (reference README.md:9)."""
    B, M, N = v.shape
    out = torch.zeros(B, M, N, dtype=v.dtype)
    for b, i, h in itertools.product(range(B), range(M), range(N)):
        out[b, i, h] = sum(a[b, i, j] * v[b, i + j - w, h] for j in range(2 * w + 1) if 0 <= i + j - w < M)
    return out


@pytest.mark.parametrize("B,M,N,w", [(1, 1, 2, 1), (2, 5, 3, 1), (1, 6, 2, 3), (1, 4, 3, 7)])
def test_brute_force_from_definition(B, M, N, w):
    q, kt, v, a, _, _ = _inputs(B, M, N, w, torch.float64, seed=7)
    torch.testing.assert_close(oracle.window_matmul_forward(q, kt, w), _readme_window(q, kt, w), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(oracle.unwindow_matmul_forward(a, v, w), _readme_unwindow(a, v, w), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("M,N,w", [(9, 4, 2), (5, 3, 8), (33, 8, 16)])
def test_all_ones_closed_form_and_exact_zeros(M, N, w):
    q = torch.ones(2, M, N)
    kt = torch.ones(2, N, M)
    a = oracle.window_matmul_forward(q, kt, w)
    mask = oracle.band_mask(M, w)
    assert torch.equal(a[:, mask], torch.full_like(a[:, mask], float(N)))
    outside = a[:, ~mask]
    assert torch.equal(outside.view(torch.int32), torch.zeros_like(outside, dtype=torch.int32))  # +0.0 bits
    # row i of the mask is [max(w-i,0), min(2w+1, M+w-i))  (reference tests/utils.py:79-81)
    for i in range(M):
        lo, hi = max(w - i, 0), min(2 * w + 1, M + w - i)
        assert mask[i].nonzero().flatten().tolist() == list(range(lo, hi))


def test_one_hot_rows_read_single_key_entries():
    M, N, w = 11, 5, 3
    kt = seeded((1, N, M), 3)
    for h in range(N):
        q = torch.zeros(1, M, N)
        q[0, :, h] = 1.0
        a = oracle.window_matmul_forward(q, kt, w)
        for i in range(M):
            for j in range(2 * w + 1):
                c = i + j - w
                expect = kt[0, h, c].item() if 0 <= c < M else 0.0
                assert a[0, i, j].item() == expect


def test_unwindow_centre_one_hot_is_identity_and_ones_is_sliding_sum():
    B, M, N, w = 2, 23, 6, 4
    v = seeded((B, M, N), 5, torch.float64)
    a = torch.zeros(B, M, 2 * w + 1, dtype=torch.float64)
    a[:, :, w] = 1.0
    assert torch.equal(oracle.unwindow_matmul_forward(a, v, w), v)
    ones = torch.ones(B, M, 2 * w + 1, dtype=torch.float64)
    cs = torch.cat([torch.zeros(B, 1, N, dtype=torch.float64), v.cumsum(1)], 1)
    lo = (torch.arange(M) - w).clamp(min=0)
    hi = (torch.arange(M) + w + 1).clamp(max=M)
    torch.testing.assert_close(oracle.unwindow_matmul_forward(ones, v, w), cs[:, hi] - cs[:, lo], rtol=1e-12, atol=1e-12)


def test_garbage_in_invalid_input_band_entries_is_ignored():
    B, M, N, w = 2, 13, 4, 5
    _, _, v, a, _, go = _inputs(B, M, N, w, torch.float32, seed=11)
    mask = oracle.band_mask(M, w)
    dirty = a.clone()
    dirty[:, ~mask] = float("nan")
    assert torch.equal(oracle.unwindow_matmul_forward(dirty, v, w), oracle.unwindow_matmul_forward(a, v, w))
    da0, dv0 = oracle.unwindow_matmul_backward(a, v, w, go)
    da1, dv1 = oracle.unwindow_matmul_backward(dirty, v, w, go)
    assert torch.equal(da0, da1) and torch.equal(dv0, dv1)
    q, kt, _, _, ga, _ = _inputs(B, M, N, w, torch.float32, seed=12)
    gd = ga.clone()
    gd[:, ~mask] = float("inf")
    for x, y in zip(oracle.window_matmul_backward(q, kt, w, ga), oracle.window_matmul_backward(q, kt, w, gd)):
        assert torch.equal(x, y)


@pytest.mark.parametrize("B,M,N,w", [(2, 17, 5, 3), (1, 8, 4, 20), (2, 40, 7, 12)])
def test_adjoint_identities(B, M, N, w):
    """<window(q,k), G> = <q, dQ> = <k, dK> and <unwindow(a,v), G> = <a*, dA> = <v, dV>."""
    q, kt, v, a, ga, go = _inputs(B, M, N, w, torch.float64, seed=21)
    mask = oracle.band_mask(M, w)
    A = oracle.window_matmul_forward(q, kt, w)
    dq, dkt = oracle.window_matmul_backward(q, kt, w, ga)
    lhs = (A * ga).sum()
    torch.testing.assert_close(lhs, (q * dq).sum(), rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(lhs, (kt * dkt).sum(), rtol=1e-10, atol=1e-10)
    O = oracle.unwindow_matmul_forward(a, v, w)
    da, dv = oracle.unwindow_matmul_backward(a, v, w, go)
    lhs = (O * go).sum()
    torch.testing.assert_close(lhs, (torch.where(mask, a, torch.zeros(())) * da).sum(), rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(lhs, (v * dv).sum(), rtol=1e-10, atol=1e-10)
    assert torch.equal(da[:, ~mask], torch.zeros_like(da[:, ~mask]))


def test_window_covering_whole_sequence_is_dense_product():
    B, M, N = 2, 10, 6
    w = M - 1
    q, kt, *_ = _inputs(B, M, N, w, torch.float64, seed=31)
    a = oracle.window_matmul_forward(q, kt, w)
    S = torch.bmm(q, kt)
    for i in range(M):
        torch.testing.assert_close(a[:, i, w - i: w - i + M], S[:, i, :], rtol=1e-12, atol=1e-12)


def test_transposed_band_identity():
    """dV = P3(A, G) equals P2(A^t, G) with A^t[c, j'] = A[c+j'-w, 2w-j'] (band transpose)."""
    B, M, N, w = 2, 19, 5, 4
    _, _, v, a, _, go = _inputs(B, M, N, w, torch.float64, seed=41)
    at = torch.zeros_like(a)
    for c in range(M):
        for jp in range(2 * w + 1):
            r = c + jp - w
            if 0 <= r < M:
                at[:, c, jp] = a[:, r, 2 * w - jp]
    _, dv = oracle.unwindow_matmul_backward(a, v, w, go)
    torch.testing.assert_close(dv, oracle.unwindow_matmul_forward(at, go, w), rtol=1e-12, atol=1e-12)


def test_shape_checks_raise():
    with pytest.raises(RuntimeError, match="Input mismatch"):
        oracle.window_matmul_forward(torch.zeros(1, 4, 3), torch.zeros(1, 4, 3), 1)
    with pytest.raises(RuntimeError, match="Input mismatch"):
        oracle.unwindow_matmul_forward(torch.zeros(1, 4, 4), torch.zeros(1, 4, 3), 1)
