"""GPU parity: every C-ABI entry point against the CPU oracle on the same seeded inputs.

Tolerances (stated by the task for this path): float32 rtol 1e-3 / atol 1e-3,
float16 / bfloat16 2e-2 (relative and absolute) against the float32 oracle on the
rounded inputs, float64 1e-9.  Out-of-sequence band entries must be bit-exact +0.0
and garbage planted in invalid entries of an input band must not reach any output.
"""
import itertools

import pytest
import torch

import wm_ctypes as abi
import oracle
from conftest import seeded

pytestmark = pytest.mark.gpu

TOL = {
    torch.float32: dict(rtol=1e-3, atol=1e-3),
    torch.float64: dict(rtol=1e-9, atol=1e-9),
    torch.float16: dict(rtol=2e-2, atol=2e-2),
    torch.bfloat16: dict(rtol=2e-2, atol=2e-2),
}

# (B, M, N, w): the reference's grid (reference tests/conftest.py:5-13) ...
REF_GRID = [(2, M, N, w) for (M, N), w in itertools.product([(1, 3), (4, 3), (16, 3), (32, 3), (16, 32)], [1, 4, 16])]
# ... plus shapes that straddle tile edges, w >= M, 2w+1 == M, N not a multiple of 8/16/32
EDGE = [
    (3, 37, 5, 6), (1, 1, 8, 3), (2, 129, 64, 4), (2, 130, 64, 64), (1, 257, 80, 33), (2, 100, 128, 49),
    (1, 300, 64, 150), (2, 65, 16, 100), (1, 513, 72, 256), (2, 96, 64, 8), (1, 200, 40, 12), (3, 64, 64, 1),
    (1, 1000, 64, 32), (2, 333, 24, 7), (3, 700, 64, 32), (1, 1100, 32, 256), (2, 900, 128, 64), (9, 260, 16, 96),
    (2, 600, 128, 16), (2, 515, 80, 20), (1, 300, 64, 7), (2, 260, 48, 28), (1, 257, 64, 8), (2, 1030, 64, 12),
    # windows that are not a multiple of 4 (band rows re-pitched on their way into LDS), odd batch strides
    (3, 201, 64, 13), (2, 150, 32, 22), (3, 141, 128, 27), (2, 90, 16, 5), (3, 171, 96, 30), (2, 400, 64, 9),
    # windows between 33 and 63 at N <= 64: band-out product on the narrow-band kernel, band-in on the wide-band ones
    (2, 300, 64, 40), (3, 201, 32, 63), (2, 150, 48, 57), (1, 700, 16, 33),
    # float32 at N <= 64, w = 12..28: narrow-band MFMA kernels for all three products
    (3, 201, 64, 12), (2, 333, 48, 17), (3, 140, 16, 28), (2, 90, 32, 21),
    # band that covers the whole sequence over many 128-row tiles (few tiles for the CUs: split tiles)
    (1, 1100, 80, 1200), (2, 777, 80, 776), (1, 1500, 64, 750),
]
CASES = REF_GRID + EDGE
DTYPES = [torch.float32, torch.bfloat16, torch.float16, torch.float64]


def make(B, M, N, w, dtype, seed=0, scale=1.0):
    q = seeded((B, M, N), seed, dtype, scale)
    k = seeded((B, M, N), seed + 1, dtype, scale)  # row-major keys; the op sees k.transpose(1, 2)
    v = seeded((B, M, N), seed + 2, dtype)
    a = seeded((B, M, 2 * w + 1), seed + 3, dtype, 0.25)
    ga = seeded((B, M, 2 * w + 1), seed + 4, dtype, 0.25)
    go = seeded((B, M, N), seed + 5, dtype)
    return q, k, v, a, ga, go


def assert_band_zeros(band, M, w):
    mask = oracle.band_mask(M, w)
    outside = band.cpu()[:, ~mask]
    ints = {2: torch.int16, 4: torch.int32, 8: torch.int64}[outside.element_size()]
    assert torch.equal(outside.view(ints), torch.zeros_like(outside, dtype=ints)), "out-of-range band entry is not +0.0"


def close(got, want, dtype):
    torch.testing.assert_close(got.cpu().to(want.dtype), want, **TOL[dtype])


@pytest.mark.parametrize("flags", [0, abi.FORCE_STRIDED, abi.NO_NARROW_BAND | abi.NO_ALIGNED_BAND],
                         ids=["auto", "strided", "wide-unaligned"])
@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("B,M,N,w", CASES)
def test_all_entry_points_match_oracle(device, B, M, N, w, dtype, flags):
    print(f"case B={B} M={M} N={N} w={w} {dtype} flags={flags}", flush=True)
    q, k, v, a, ga, go = make(B, M, N, w, dtype)
    kt = k.transpose(1, 2)
    mask = oracle.band_mask(M, w)
    # garbage in the invalid entries of the input bands must be ignored
    a_dirty, ga_dirty = a.clone(), ga.clone()
    a_dirty[:, ~mask] = float("nan")
    ga_dirty[:, ~mask] = float("inf")
    dq, dk, dv, da_, dga, dgo = (t.to(device) for t in (q, k, v, a_dirty, ga_dirty, go))
    dkt = dk.transpose(1, 2)

    got = abi.window_forward(dq, dkt, w, flags)
    close(got, oracle.window_matmul_forward(q, kt, w), dtype)
    assert_band_zeros(got, M, w)

    gq, gk = abi.window_backward(dq, dkt, w, dga, flags)
    rq, rk = oracle.window_matmul_backward(q, kt, w, ga)
    close(gq, rq, dtype)
    close(gk, rk, dtype)

    got = abi.unwindow_forward(da_, dv, w, flags)
    close(got, oracle.unwindow_matmul_forward(a, v, w), dtype)

    gA, gV = abi.unwindow_backward(da_, dv, w, dgo, flags)
    rA, rV = oracle.unwindow_matmul_backward(a, v, w, go)
    close(gA, rA, dtype)
    close(gV, rV, dtype)
    assert_band_zeros(gA, M, w)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_key_layouts_and_strided_views(device, dtype):
    """K as contiguous (B,N,M), as a transposed view, and head-major non-contiguous q/k/v
    (reference tests/utils.py:38-44) all give the same numbers."""
    B, H, M, N, w = 2, 3, 70, 16, 9
    base = [seeded((B, M, H * N), s, dtype).to(device) for s in (1, 2, 3)]
    q, k, v = (t.view(B, M, H, N).transpose(1, 2).reshape(B * H, M, N) for t in base)  # copies, row-major
    qv, kv, vv = (t.view(B, M, H, N).transpose(1, 2) for t in base)  # non-contiguous views
    want = abi.window_forward(q, k.transpose(1, 2), w)
    # contiguous (B,N,M) keys
    got = abi.window_forward(q, k.transpose(1, 2).contiguous(), w)
    torch.testing.assert_close(got, want, **TOL[dtype])
    # per-head strided views: batch stride is not expressible for (B,H) jointly, so go head by head
    for h in range(H):
        got_h = abi.window_forward(qv[:, h], kv[:, h].transpose(1, 2), w)
        torch.testing.assert_close(got_h, want.view(B, H, M, -1)[:, h], **TOL[dtype])
        o_h = abi.unwindow_forward(want.view(B, H, M, -1)[:, h].contiguous(), vv[:, h], w)
        o = abi.unwindow_forward(want, v, w)
        torch.testing.assert_close(o_h, o.view(B, H, M, N)[:, h], **TOL[dtype])


def test_skipping_one_gradient(device):
    B, M, N, w = 2, 50, 16, 5
    q, k, v, a, ga, go = (t.to(device) for t in make(B, M, N, w, torch.float32))
    kt = k.transpose(1, 2)
    gq, gk = abi.window_backward(q, kt, w, ga)
    gq_only, none = abi.window_backward(q, kt, w, ga, want_k=False)
    assert none is None and torch.equal(gq_only, gq)
    none, gk_only = abi.window_backward(q, kt, w, ga, want_q=False)
    assert none is None and torch.equal(gk_only, gk)
    gA, gV = abi.unwindow_backward(a, v, w, go)
    gA_only, _ = abi.unwindow_backward(a, v, w, go, want_v=False)
    _, gV_only = abi.unwindow_backward(a, v, w, go, want_a=False)
    assert torch.equal(gA_only, gA) and torch.equal(gV_only, gV)


def test_runs_on_a_side_stream(device):
    B, M, N, w = 2, 64, 32, 8
    q, k, *_ = (t.to(device) for t in make(B, M, N, w, torch.float32))
    want = abi.window_forward(q, k.transpose(1, 2), w)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        got = abi.window_forward(q, k.transpose(1, 2), w)
    s.synchronize()
    assert torch.equal(got, want)


@pytest.mark.parametrize("B", [7, 8, 9, 12, 17, 23])
@pytest.mark.parametrize("dtype,N,w", [(torch.bfloat16, 64, 64), (torch.bfloat16, 64, 8), (torch.float16, 128, 2),
                                       (torch.float32, 80, 40), (torch.float32, 32, 16), (torch.float32, 64, 3)],
                         ids=["wide", "narrow", "vector", "f32-mfma", "f32-narrow", "f32-vector"])
def test_batch_counts_around_multiples_of_eight(device, B, dtype, N, w):
    """Workgroups are dealt to the 8 XCDs by batch element for full groups of 8 and by ranges of tiles
    for the elements left over: every (batch element, block) must be computed exactly once, whatever B."""
    M = 300
    print(f"case B={B} {dtype} N={N} w={w}", flush=True)
    q, k, v, a, ga, go = (t.to(device) for t in make(B, M, N, w, dtype, seed=40))
    kt = k.transpose(1, 2)
    tol = dict(rtol=1e-3, atol=1e-3) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    got, want = [], []
    for flags, res in ((0, got), (abi.FORCE_STRIDED, want)):
        res.append(abi.window_forward(q, kt, w, flags))
        res.extend(abi.window_backward(q, kt, w, ga, flags))
        res.append(abi.unwindow_forward(a, v, w, flags))
        res.extend(abi.unwindow_backward(a, v, w, go, flags))
    for x, y in zip(got, want):
        torch.testing.assert_close(x.float(), y.float(), **tol)
    if dtype != torch.float32:
        scale = N ** -0.5
        o, lse = abi.attention_forward(q, k, v, w, scale)
        grads = abi.attention_backward(q, k, v, o, lse, go, w, scale)
        o1, lse1 = abi.attention_forward(q[B - 1:], k[B - 1:], v[B - 1:], w, scale)
        g1 = abi.attention_backward(q[B - 1:], k[B - 1:], v[B - 1:], o1, lse1, go[B - 1:], w, scale)
        assert torch.equal(o[B - 1:], o1) and torch.equal(lse[B - 1:], lse1)
        for x, y in zip(grads, g1):
            assert torch.equal(x[B - 1:], y)
