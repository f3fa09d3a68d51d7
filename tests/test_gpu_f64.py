"""float64: the register-blocked tile kernels against the strided kernels and the oracle.

The tile kernels sum in the same order as the strided ones (ascending contraction index, one
rounding per term where the compiler fuses the multiply-add), so the two agree to the last few
bits: the tolerance here is 1e-12 where the oracle comparison of test_gpu_parity uses 1e-9.
The layouts are the ones the reference's callers produce (reference tests/utils.py:38-44,
cuda/window_matmul_cuda.cu:236, 285): keys stored (B,N,M), head-major views of a fused
projection, bands cut out of a wider tensor, results written into slices.
"""
import pytest
import torch

import oracle
import wm_ctypes as abi
from conftest import seeded

pytestmark = pytest.mark.gpu

F64 = torch.float64
TIGHT = dict(rtol=1e-12, atol=1e-12)
# (B, M, N, w): tile edges (64 rows, 64 columns, stages of 16), one row, w >= M, widths around 64
SHAPES = [(3, 1000, 72, 100), (2, 2048, 64, 256), (1, 64, 64, 0), (2, 65, 1, 3), (1, 1, 200, 5), (2, 127, 65, 200),
          (5, 300, 130, 17), (1, 4096, 16, 1), (2, 513, 48, 64)]


def operands(B, M, N, w, device):
    q, k, v, go = (seeded((B, M, N), 300 + s, F64).to(device) for s in range(4))
    a, ga = (seeded((B, M, 2 * w + 1), 310 + s, F64, 0.25).to(device) for s in range(2))
    return q, k, v, go, a, ga


def all_six(q, kt, v, go, a, ga, w, flags):
    band = abi.window_forward(q, kt, w, flags)
    gq, gk = abi.window_backward(q, kt, w, ga, flags)
    o = abi.unwindow_forward(a, v, w, flags)
    gA, gV = abi.unwindow_backward(a, v, w, go, flags)
    return dict(band=band, gq=gq, gk=gk, o=o, gA=gA, gV=gV)


def test_kernel_choice_is_the_tile_family():
    L = abi.lib()
    for op in (1, 2, 3):
        for fast in (0, 1):
            assert L.wm_kernel_choice(op, 2, 300, 72, 17, abi.DTYPES[F64], fast, 0) == f"f64_tile_p{op}".encode()


@pytest.mark.parametrize("B,M,N,w", SHAPES)
def test_tiles_agree_with_strided_kernels(device, B, M, N, w):
    print(f"case B={B} M={M} N={N} w={w}", flush=True)
    q, k, v, go, a, ga = operands(B, M, N, w, device)
    kt = k.transpose(1, 2)
    got, want = all_six(q, kt, v, go, a, ga, w, 0), all_six(q, kt, v, go, a, ga, w, abi.FORCE_STRIDED)
    for name in want:
        torch.testing.assert_close(got[name], want[name], **TIGHT, msg=lambda m, n=name: f"{n}: {m}")
    mask = oracle.band_mask(M, w).to(device)
    for name in ("band", "gA"):
        outside = got[name][:, ~mask].view(torch.int64)
        assert int(outside.abs().max() if outside.numel() else 0) == 0, f"{name}: out-of-sequence entry is not +0.0"


def test_layouts(device):
    """Stored (B,N,M) keys, head-major views, a band cut out of a wider tensor, results into slices."""
    B, H, M, N, w = 2, 3, 210, 24, 37
    W = 2 * w + 1
    fused = [seeded((B, M, H * N), 320 + s, F64).to(device) for s in range(4)]
    rows = [t.view(B, M, H, N).transpose(1, 2).reshape(B * H, M, N) for t in fused]  # row-major copies
    views = [t.view(B, M, H, N).transpose(1, 2) for t in fused]                      # (B, H, M, N) views
    wide = seeded((B * H, M, W + 11), 330, F64, 0.25).to(device)
    a_view, a = wide[:, :, 5:5 + W], wide[:, :, 5:5 + W].contiguous()
    q, k, v, go = rows

    want = all_six(q, k.transpose(1, 2), v, go, a, a, w, abi.FORCE_STRIDED)

    # keys stored (B,N,M): rows of the key operand are one element apart
    stored = k.transpose(1, 2).contiguous()
    torch.testing.assert_close(abi.window_forward(q, stored, w), want["band"], **TIGHT)
    gq, gk = abi.window_backward(q, stored, w, a_view)
    torch.testing.assert_close(gq, want["gq"], **TIGHT)
    torch.testing.assert_close(gk, want["gk"], **TIGHT)

    # non-contiguous band operand
    torch.testing.assert_close(abi.unwindow_forward(a_view, v, w), want["o"], **TIGHT)
    gA, gV = abi.unwindow_backward(a_view, v, w, go)
    torch.testing.assert_close(gA, want["gA"], **TIGHT)
    torch.testing.assert_close(gV, want["gV"], **TIGHT)

    # band written into a slice of a wider tensor: the columns beside it stay as they were
    target = torch.full((B * H, M, W + 4), 7.0, dtype=F64, device=device)
    abi.window_forward(q, k.transpose(1, 2), w, out=target[:, :, 2:2 + W])
    torch.testing.assert_close(target[:, :, 2:2 + W], want["band"], **TIGHT)
    assert bool((target[:, :, :2] == 7.0).all()) and bool((target[:, :, 2 + W:] == 7.0).all())

    # head-major views, one head at a time (the joint (B,H) batch stride is not expressible)
    qv, kv, vv, gov = views
    for h in range(H):
        pick = lambda t: t.view(B, H, *t.shape[1:])[:, h]  # noqa: E731
        torch.testing.assert_close(abi.window_forward(qv[:, h], kv[:, h].transpose(1, 2), w), pick(want["band"]), **TIGHT)
        torch.testing.assert_close(abi.unwindow_forward(pick(a).contiguous(), vv[:, h], w), pick(want["o"]), **TIGHT)
        gA_h, gV_h = abi.unwindow_backward(pick(a).contiguous(), vv[:, h], w, gov[:, h])
        torch.testing.assert_close(gA_h, pick(want["gA"]), **TIGHT)
        torch.testing.assert_close(gV_h, pick(want["gV"]), **TIGHT)


def test_invalid_band_entries_are_never_read_as_numbers(device):
    """NaN and Inf planted outside the sequence in both input bands leave every result finite and equal."""
    B, M, N, w = 2, 150, 40, 90
    q, k, v, go, a, ga = operands(B, M, N, w, device)
    mask = oracle.band_mask(M, w).to(device)
    a_dirty, ga_dirty = a.clone(), ga.clone()
    a_dirty[:, ~mask] = float("nan")
    ga_dirty[:, ~mask] = float("inf")
    kt = k.transpose(1, 2)
    clean, dirty = all_six(q, kt, v, go, a, ga, w, 0), all_six(q, kt, v, go, a_dirty, ga_dirty, w, 0)
    for name in clean:
        assert torch.equal(clean[name], dirty[name]), name


def test_against_the_oracle_at_a_wide_head(device):
    B, M, N, w = 2, 180, 150, 23
    q, k, v, go, a, ga = operands(B, M, N, w, device)
    kt = k.transpose(1, 2)
    got = all_six(q, kt, v, go, a, ga, w, 0)
    cpu = lambda t: t.cpu()  # noqa: E731
    want_q, want_k = oracle.window_matmul_backward(cpu(q), cpu(kt), w, cpu(ga))
    want_a, want_v = oracle.unwindow_matmul_backward(cpu(a), cpu(v), w, cpu(go))
    tol = dict(rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(cpu(got["band"]), oracle.window_matmul_forward(cpu(q), cpu(kt), w), **tol)
    torch.testing.assert_close(cpu(got["gq"]), want_q, **tol)
    torch.testing.assert_close(cpu(got["gk"]), want_k, **tol)
    torch.testing.assert_close(cpu(got["o"]), oracle.unwindow_matmul_forward(cpu(a), cpu(v), w), **tol)
    torch.testing.assert_close(cpu(got["gA"]), want_a, **tol)
    torch.testing.assert_close(cpu(got["gV"]), want_v, **tol)
