"""GPU parity of the band softmax (C ABI and Python function) against the float64 numpy
oracle on the same seeded inputs, and against the torch chain the reference's callers
write (reference tests/test_attention.py:57-63).

Tolerances: float32 rtol 1e-4 / atol 1e-6 (tighter than the 1e-3 the path allows), float16 /
bfloat16 2e-2 against the oracle on the rounded inputs, float64 1e-12.  Masked entries must
be bit-exact +0.0."""
import math

import numpy as np
import pytest
import torch

import wm_ctypes as abi
from oracle import softmax_oracle as so
from conftest import seeded

pytestmark = pytest.mark.gpu

TOL = {
    torch.float32: dict(rtol=1e-4, atol=1e-6),
    torch.float64: dict(rtol=1e-12, atol=1e-14),
    torch.float16: dict(rtol=2e-2, atol=2e-2),
    torch.bfloat16: dict(rtol=2e-2, atol=2e-2),
}
# (B, M, w): single element rows, rows shorter than a chunk, ragged last workgroup, rows that stay in
# registers (<= 1280), rows re-read from LDS (1281, 3001), rows too long for LDS (strided kernel)
CASES = [
    (1, 1, 0), (3, 5, 0), (2, 5, 1), (3, 17, 3), (2, 100, 8), (5, 1000, 8), (2, 64, 16), (3, 129, 33), (2, 300, 128),
    (1, 200, 256), (7, 37, 256), (2, 77, 640), (1, 40, 1500), (1, 3, 9000), (1, 2, 20000),
]
DTYPES = [torch.float32, torch.bfloat16, torch.float16, torch.float64]


def f64(t):
    return t.detach().cpu().to(torch.float64).numpy()


def close(got, want, dtype):
    torch.testing.assert_close(got.cpu().to(torch.float64), torch.from_numpy(want), **TOL[dtype])


def assert_masked_zero(t, M, w):
    outside = t.cpu()[:, ~torch.from_numpy(so.valid_mask(M, w))]
    ints = {2: torch.int16, 4: torch.int32, 8: torch.int64}[outside.element_size()]
    assert torch.equal(outside.view(ints), torch.zeros_like(outside, dtype=ints)), "masked entry is not +0.0"


@pytest.mark.parametrize("flags", [0, abi.FORCE_STRIDED], ids=["auto", "strided"])
@pytest.mark.parametrize("mask", [False, True], ids=["zero_filled", "masked"])
@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%d_M%d_w%d" % c)
def test_forward_and_backward_match_oracle(device, case, dtype, mask, flags):
    B, M, w = case
    W = 2 * w + 1
    scale = 1.0 / math.sqrt(64)
    a = seeded((B, M, W), 11, dtype, 4.0)
    gp = seeded((B, M, W), 12, dtype)
    if mask:  # whatever sits in masked entries must not matter
        keep = torch.from_numpy(so.valid_mask(M, w))
        a[:, ~keep] = float("nan")
        gp[:, ~keep] = float("inf")
    want_p = so.band_softmax_forward(f64(a), scale, mask)
    p = abi.band_softmax_forward(a.to(device), scale, mask, flags)
    close(p, want_p, dtype)
    # backward from the probabilities the kernel itself stored (what autograd hands it)
    want_g = so.band_softmax_backward(f64(p), f64(gp), scale, mask)
    g = abi.band_softmax_backward(p, gp.to(device), scale, mask, flags)
    close(g, want_g, dtype)
    if mask:
        assert_masked_zero(p, M, w)
        assert_masked_zero(g, M, w)
    name = abi.lib().wm_band_softmax_kernel_choice(w, abi.DTYPES[dtype], 1, 0, flags).decode()
    staged = flags == 0 and dtype != torch.float64 and W * a.element_size() <= 65536 - 32
    assert name == ("staged_softmax" if staged else "strided_softmax")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("case", [(3, 129, 33), (5, 1000, 8), (1, 40, 1500)], ids=lambda c: "B%d_M%d_w%d" % c)
def test_in_place(device, case, dtype):
    B, M, w = case
    a = seeded((B, M, 2 * w + 1), 13, dtype, 2.0).to(device)
    gp = seeded((B, M, 2 * w + 1), 14, dtype).to(device)
    p = abi.band_softmax_forward(a, 0.5)
    buf = a.clone()
    assert abi.band_softmax_forward(buf, 0.5, out=buf) is buf
    assert torch.equal(buf, p)
    g = abi.band_softmax_backward(p, gp, 0.5)
    buf = gp.clone()
    abi.band_softmax_backward(p, buf, 0.5, out=buf)
    assert torch.equal(buf, g)
    buf = p.clone()
    abi.band_softmax_backward(buf, gp, 0.5, out=buf)
    assert torch.equal(buf, g)


def test_offset_and_strided_operands(device):
    """A base pointer that is not 16-byte aligned, and a non-contiguous band: strided kernel, same values."""
    B, M, w = 2, 50, 9
    W = 2 * w + 1
    big = seeded((B * M * W + 3,), 15, torch.float32).to(device)
    a = big[3:].view(B, M, W)
    want = so.band_softmax_forward(f64(a), 1.0)
    close(abi.band_softmax_forward(a, 1.0), want, torch.float32)
    wide = seeded((B, M, W + 5), 16, torch.float32).to(device)
    a = wide[:, :, 2:2 + W]
    close(abi.band_softmax_forward(a, 1.0), so.band_softmax_forward(f64(a), 1.0), torch.float32)


@pytest.mark.parametrize("mask", [False, True], ids=["zero_filled", "masked"])
def test_python_function_and_autograd(device, mask):
    from window_matmul import band_softmax

    batch, heads, M, w = 2, 3, 70, 12
    a0 = seeded((batch, heads, M, 2 * w + 1), 17, torch.float32).to(device)
    g0 = seeded((batch, heads, M, 2 * w + 1), 18, torch.float32).to(device)
    keep = torch.from_numpy(so.valid_mask(M, w)).to(device)
    res = {}
    for name in ("torch", "ours"):
        a = a0.clone().requires_grad_(True)
        if name == "torch":
            x = a * 0.25
            p = torch.softmax(x.masked_fill(~keep, float("-inf")) if mask else x, -1)
        else:
            p = band_softmax(a, 0.25, mask)
        p.backward(g0)
        res[name] = (p.detach(), a.grad)
    assert res["ours"][0].shape == a0.shape
    for x, y in zip(res["ours"], res["torch"]):
        torch.testing.assert_close(x, y, rtol=1e-5, atol=1e-7)
    # default scale is 1, the result of a 2-D input keeps its shape
    torch.testing.assert_close(band_softmax(a0[0, 0]), torch.softmax(a0[0, 0], -1), rtol=1e-5, atol=1e-7)
    with pytest.raises(RuntimeError, match="Input mismatch"):
        band_softmax(a0[..., :-1])
    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        band_softmax(a0.cpu())


def test_gradcheck_float64(device):
    from window_matmul import band_softmax

    a = seeded((2, 6, 7), 19, torch.float64).to(device).requires_grad_(True)
    assert torch.autograd.gradcheck(lambda t: band_softmax(t, 0.7, False), (a,), eps=1e-6, atol=1e-6)
    assert torch.autograd.gradcheck(lambda t: band_softmax(t, 0.7, True), (a,), eps=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_attention_chain_with_band_softmax(device, dtype):
    """window_matmul -> band_softmax -> unwindow_matmul equals the same chain with torch.softmax
    (reference tests/test_attention.py:57-63), outputs and input gradients."""
    from window_matmul import band_softmax, unwindow_matmul, window_matmul

    B, M, N, w = 4, 300, 64, 40
    q0, k0, v0 = (seeded((B, M, N), s, dtype).to(device) for s in (21, 22, 23))
    go = seeded((B, M, N), 24, dtype).to(device)
    res = {}
    for name in ("torch", "ours"):
        q, k, v = (t.clone().requires_grad_(True) for t in (q0, k0, v0))
        att = window_matmul(q, k.transpose(-1, -2), w)
        if name == "torch":
            probs = torch.softmax(att / math.sqrt(N), -1)
        else:
            probs = band_softmax(att, 1.0 / math.sqrt(N))
        out = unwindow_matmul(probs, v, w)
        out.backward(go)
        res[name] = (out.detach(), q.grad, k.grad, v.grad)
    tol = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    for x, y in zip(res["ours"], res["torch"]):
        torch.testing.assert_close(x.float(), y.float(), **tol)
