"""Tensors whose flat element indices do not fit 32 bits, on the GPU.

Extents stay below 2^31 but B*M*(2w+1) or B*M*N does not, or M*(2w+1) within one batch element.
Checking such sizes against the CPU oracle would take hours, so the check is a size-independent
property: every product is local (row i of a result depends on rows i-w..i+w of its operands and
on nothing of other batch elements), so the same call on a contiguous slice that holds the far
end of the big tensors -- the last batch element, or the last rows of the sequence -- must
reproduce the far end of the big result.  The small call has small offsets; the kernels behind it
are checked against the oracle elsewhere.  Tolerance 2e-2 of the largest magnitude (16-bit
storage; the two calls may differ in chunk alignment, hence in summation order).
"""
import pytest
import torch

import wm_ctypes as abi

pytestmark = pytest.mark.gpu

LIMIT = 2 ** 31


def _close(got, want, what):
    got, want = got.float(), want.float()
    assert torch.isfinite(got).all(), what
    err = (got - want).abs().max().item()
    assert err <= 2e-2 * max(1.0, want.abs().max().item()), f"{what}: max error {err}"


def _rand(shape, dtype, device, seed, scale=1.0):
    g = torch.Generator(device=device).manual_seed(seed)
    t = torch.empty(shape, dtype=dtype, device=device)
    t.normal_(0.0, scale, generator=g)
    return t


def _all_products(q, k, v, go, a, w, flags=0):
    """The six banded products through the C ABI (k row-major, consumed in place)."""
    att = abi.window_forward(q, k.transpose(1, 2), w, flags)
    out = abi.unwindow_forward(a, v, w, flags)
    ga, gv = abi.unwindow_backward(a, v, w, go, flags)
    gq, gk = abi.window_backward(q, k.transpose(1, 2), w, a, flags)
    return dict(window_fwd=att, unwindow_fwd=out, grad_a=ga, grad_v=gv, grad_q=gq, grad_k=gk.transpose(1, 2))


# (B, M, N, w, dtype, flags): which index passes 2^31, and which kernels take the case
BATCH_CASES = [
    pytest.param(3, 1 << 20, 16, 512, torch.bfloat16, 0, id="band-wide-w512"),    # band 3.2 G elements
    pytest.param(9, 1 << 22, 16, 30, torch.bfloat16, 0, id="band-narrow-w30"),    # band 2.3 G, re-pitched LDS image
    pytest.param(5, 1 << 22, 128, 2, torch.float16, 0, id="rows-vector-w2"),      # q, k, v 2.7 G elements
    pytest.param(5, 1 << 22, 128, 8, torch.bfloat16, 0, id="rows-narrow-w8"),
    pytest.param(9, 1 << 22, 64, 4, torch.float32, 0, id="rows-vector-f32-w4"),   # q, k, v 2.4 G elements
    pytest.param(9, 1 << 22, 64, 20, torch.float32, 0, id="rows-mfma-f32-w20"),
    pytest.param(5, 1 << 22, 128, 2, torch.float16, abi.FORCE_STRIDED, id="rows-strided-w2"),
    pytest.param(3, 1 << 20, 20, 512, torch.bfloat16, 0, id="band-tile-bf16-n20"),  # head width no tuned kernel takes
    pytest.param(3, 1 << 20, 16, 400, torch.float64, 0, id="band-tile-f64-w400"),   # band 2.5 G elements, 20 GB
]


@pytest.mark.parametrize("B,M,N,w,dtype,flags", BATCH_CASES)
def test_last_batch_element_of_a_large_tensor(device, B, M, N, w, dtype, flags):
    W = 2 * w + 1
    assert max(B * M * W, B * M * N) > LIMIT
    q, k, v, go = (_rand((B, M, N), dtype, device, s) for s in (1, 2, 3, 4))
    a = _rand((B, M, W), dtype, device, 5, 0.2)
    big = _all_products(q, k, v, go, a, w, flags)
    last = _all_products(*(t[B - 1:] for t in (q, k, v, go, a)), w, flags)
    for name in big:
        _close(big[name][B - 1:], last[name], name)
    del big, last, q, k, v, go, a
    torch.cuda.empty_cache()


def test_last_rows_of_a_long_sequence(device):
    """One batch element whose band alone has more than 2^31 elements."""
    M, N, w, dtype = (1 << 21) + 1000, 16, 512, torch.bfloat16
    W, tail = 2 * w + 1, 8192
    assert M * W > LIMIT
    q, k, v, go = (_rand((1, M, N), dtype, device, s) for s in (11, 12, 13, 14))
    a = _rand((1, M, W), dtype, device, 15, 0.2)
    big = _all_products(q, k, v, go, a, w)
    s0 = M - tail
    sub = _all_products(*(t[:, s0:] for t in (q, k, v, go, a)), w)
    for name in big:  # rows further than w from the cut see the same neighbours in both calls
        _close(big[name][:, s0 + w:], sub[name][:, w:], name)
    del big, sub, q, k, v, go, a
    torch.cuda.empty_cache()


def test_band_softmax_and_attention_on_a_large_band(device):
    B, M, N, w, dtype = 3, 1 << 20, 16, 512, torch.bfloat16
    W = 2 * w + 1
    assert B * M * W > LIMIT
    a = _rand((B, M, W), dtype, device, 21)
    gp = _rand((B, M, W), dtype, device, 22)
    p = abi.band_softmax_forward(a, 0.5, True)
    ga = abi.band_softmax_backward(p, gp, 0.5, True)
    _close(p[B - 1:], abi.band_softmax_forward(a[B - 1:], 0.5, True), "band_softmax forward")
    _close(ga[B - 1:], abi.band_softmax_backward(p[B - 1:], gp[B - 1:], 0.5, True), "band_softmax backward")
    del a, gp, p, ga
    torch.cuda.empty_cache()
    # fused attention never forms the band; its large index is B*M*N
    B, M, N, w = 5, 1 << 22, 128, 16
    assert B * M * N > LIMIT
    q, k, v, go = (_rand((B, M, N), dtype, device, s) for s in (31, 32, 33, 34))
    o, lse = abi.attention_forward(q, k, v, w, 0.1, False)
    gq, gk, gv = abi.attention_backward(q, k, v, o, lse, go, w, 0.1)
    ql, kl, vl, gol = (t[B - 1:] for t in (q, k, v, go))
    o1, lse1 = abi.attention_forward(ql, kl, vl, w, 0.1, False)
    g1 = abi.attention_backward(ql, kl, vl, o1, lse1, gol, w, 0.1)
    _close(o[B - 1:], o1, "attention output")
    for name, x, y in zip(("grad_q", "grad_k", "grad_v"), (gq, gk, gv), g1):
        _close(x[B - 1:], y, name)


@pytest.mark.parametrize("shape", [(1, 4_000_037, 64, 8), (2, 1_500_000, 48, 64)], ids=lambda s: "B%d_M%d_N%d_w%d" % s)
def test_one_kernel_attention_backward_on_a_long_sequence(device, shape):
    """The one-kernel backward of the fused attention addresses a batch element with 32-bit byte offsets
    (up to 2^31 bytes per tensor): at sequences of millions of rows it must give what the two-kernel
    form gives, also in the last rows, where the offsets are largest."""
    B, M, N, w = shape
    g = torch.Generator(device=device).manual_seed(1)
    q, k, v, go = (torch.randn(B, M, N, device=device, generator=g).to(torch.bfloat16) for _ in range(4))
    scale = N ** -0.5
    o, lse = abi.attention_forward(q, k, v, w, scale)
    one = abi.attention_backward(q, k, v, o, lse, go, w, scale)
    two = abi.attention_backward(q, k, v, o, lse, go, w, scale, flags=abi.NO_NARROW_BAND)
    for x, y in zip(one, two):
        assert bool(torch.isfinite(x).all())
        torch.testing.assert_close(x[:, -1000:].float(), y[:, -1000:].float(), rtol=2e-2, atol=2e-2)
        torch.testing.assert_close(x[:, ::997].float(), y[:, ::997].float(), rtol=2e-2, atol=2e-2)
