"""The tile kernels (float64, and every layout or head width the tuned kernels decline in the
other storage types) against the strided kernels and the oracle.

Both families sum in ascending order of the contraction index, the tile kernels four terms per
matrix instruction, in float64 for float64 storage and in float32 otherwise, and round once: the
tolerances are 1e-12 for float64 (test_gpu_parity compares with the oracle at 1e-9), 1e-4 for
float32 and one unit in the last place of the 16-bit types.
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
DTYPES = [torch.float64, torch.float32, torch.bfloat16, torch.float16]
TIGHT = {
    torch.float64: dict(rtol=1e-12, atol=1e-12),
    torch.float32: dict(rtol=1e-4, atol=1e-4),
    torch.bfloat16: dict(rtol=1e-2, atol=1e-2),
    torch.float16: dict(rtol=2e-3, atol=2e-3),
}
# (B, M, N, w): tile edges (64 rows, 64 columns, stages of 16), one row, w >= M, head widths that no
# tuned kernel takes (not a multiple of 8, beyond 128)
SHAPES = [(3, 1000, 71, 100), (1, 64, 63, 0), (2, 65, 1, 3), (1, 1, 200, 5), (2, 127, 65, 200), (5, 300, 130, 17),
          (2, 513, 47, 64), (1, 2100, 3, 4)]
F64_SHAPES = [(2, 2048, 64, 256), (1, 4096, 16, 1), (2, 513, 48, 64)]  # widths the other types have tuned kernels for
CASES = [(s, d) for d in DTYPES for s in SHAPES] + [(s, F64) for s in F64_SHAPES]


def operands(B, M, N, w, device, dtype=F64):
    q, k, v, go = (seeded((B, M, N), 300 + s, dtype).to(device) for s in range(4))
    a, ga = (seeded((B, M, 2 * w + 1), 310 + s, dtype, 0.25).to(device) for s in range(2))
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
            assert L.wm_kernel_choice(op, 2, 300, 72, 17, abi.DTYPES[F64], fast, 0) == f"tile_p{op}".encode()
        for dtype in DTYPES[1:]:
            assert L.wm_kernel_choice(op, 2, 300, 64, 17, abi.DTYPES[dtype], 0, 0) == f"tile_p{op}".encode()  # layout
            assert L.wm_kernel_choice(op, 2, 300, 64, 17, abi.DTYPES[dtype], 1, 0) != f"tile_p{op}".encode()


@pytest.mark.parametrize("shape,dtype", CASES, ids=lambda x: str(x).replace("torch.", "").replace(" ", ""))
def test_tiles_agree_with_strided_kernels(device, shape, dtype):
    B, M, N, w = shape
    print(f"case B={B} M={M} N={N} w={w} {dtype}", flush=True)
    for op in (1, 2, 3):
        assert abi.lib().wm_kernel_choice(op, B, M, N, w, abi.DTYPES[dtype], 1, 0) == f"tile_p{op}".encode()
    q, k, v, go, a, ga = operands(B, M, N, w, device, dtype)
    kt = k.transpose(1, 2)
    got, want = all_six(q, kt, v, go, a, ga, w, 0), all_six(q, kt, v, go, a, ga, w, abi.FORCE_STRIDED)
    for name in want:
        torch.testing.assert_close(got[name], want[name], **TIGHT[dtype], msg=lambda m, n=name: f"{n}: {m}")
    mask = oracle.band_mask(M, w).to(device)
    ints = {2: torch.int16, 4: torch.int32, 8: torch.int64}[got["band"].element_size()]
    for name in ("band", "gA"):
        outside = got[name][:, ~mask].view(ints)
        assert int(outside.abs().max() if outside.numel() else 0) == 0, f"{name}: out-of-sequence entry is not +0.0"


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
def test_layouts(device, dtype):
    """Stored (B,N,M) keys, head-major views, a band cut out of a wider tensor, results into slices."""
    B, H, M, N, w = 2, 3, 210, 24, 37
    W = 2 * w + 1
    tol = TIGHT[dtype]
    fused = [seeded((B, M, H * N), 320 + s, dtype).to(device) for s in range(4)]
    rows = [t.view(B, M, H, N).transpose(1, 2).reshape(B * H, M, N) for t in fused]  # row-major copies
    views = [t.view(B, M, H, N).transpose(1, 2) for t in fused]                      # (B, H, M, N) views
    wide = seeded((B * H, M, W + 11), 330, dtype, 0.25).to(device)
    a_view, a = wide[:, :, 5:5 + W], wide[:, :, 5:5 + W].contiguous()
    q, k, v, go = rows

    want = all_six(q, k.transpose(1, 2), v, go, a, a, w, abi.FORCE_STRIDED)

    # keys stored (B,N,M): rows of the key operand are one element apart
    stored = k.transpose(1, 2).contiguous()
    torch.testing.assert_close(abi.window_forward(q, stored, w), want["band"], **tol)
    gq, gk = abi.window_backward(q, stored, w, a_view)
    torch.testing.assert_close(gq, want["gq"], **tol)
    torch.testing.assert_close(gk, want["gk"], **tol)

    # non-contiguous band operand
    torch.testing.assert_close(abi.unwindow_forward(a_view, v, w), want["o"], **tol)
    gA, gV = abi.unwindow_backward(a_view, v, w, go)
    torch.testing.assert_close(gA, want["gA"], **tol)
    torch.testing.assert_close(gV, want["gV"], **tol)

    # band written into a slice of a wider tensor: the columns beside it stay as they were
    target = torch.full((B * H, M, W + 4), 7.0, dtype=dtype, device=device)
    abi.window_forward(q, k.transpose(1, 2), w, out=target[:, :, 2:2 + W])
    torch.testing.assert_close(target[:, :, 2:2 + W], want["band"], **tol)
    assert bool((target[:, :, :2] == 7.0).all()) and bool((target[:, :, 2 + W:] == 7.0).all())

    # head-major views, one head at a time (the joint (B,H) batch stride is not expressible)
    qv, kv, vv, gov = views
    for h in range(H):
        pick = lambda t: t.view(B, H, *t.shape[1:])[:, h]  # noqa: E731
        torch.testing.assert_close(abi.window_forward(qv[:, h], kv[:, h].transpose(1, 2), w), pick(want["band"]), **tol)
        torch.testing.assert_close(abi.unwindow_forward(pick(a).contiguous(), vv[:, h], w), pick(want["o"]), **tol)
        gA_h, gV_h = abi.unwindow_backward(pick(a).contiguous(), vv[:, h], w, gov[:, h])
        torch.testing.assert_close(gA_h, pick(want["gA"]), **tol)
        torch.testing.assert_close(gV_h, pick(want["gV"]), **tol)


@pytest.mark.parametrize("dtype", [torch.float64, torch.bfloat16], ids=["float64", "bfloat16"])
def test_invalid_band_entries_are_never_read_as_numbers(device, dtype):
    """NaN and Inf planted outside the sequence in both input bands leave every result finite and equal."""
    B, M, N, w = 2, 150, 41, 90
    q, k, v, go, a, ga = operands(B, M, N, w, device, dtype)
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
