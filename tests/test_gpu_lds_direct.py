"""The kernels that load their tiles straight into LDS, against the register-staged kernels and the oracle.

The wide-band family has a second implementation of each product whose chunks never pass through
registers (band-out product at N = 128 with whole-line column groups; band-in products at every
head width, for any window as long as the band is 4-byte aligned).  ``WM_FLAG_NO_LDS_DIRECT``
switches them off, so every shape here runs both ways: the results must agree within the 16-bit
tolerance (rtol = atol = 2e-2; bit for bit where the order of the sums is the same: band-out
product, and band-in product when the window is a multiple of 4), and both must match the CPU
oracle.  Every shape here has fewer tiles than half the CUs, so the band-in products with N a multiple
of 32 run with one workgroup per block of 32 or 64 columns of Y.  Shapes cover ragged sequence ends, sequences shorter than a tile, batch elements whose band does not start on a 128-byte line, operands with padded rows and
batches, and invalid band entries filled with NaN.
"""
import pytest
import torch

import oracle
import wm_ctypes as abi
from conftest import seeded

pytestmark = pytest.mark.gpu

TOL = dict(rtol=2e-2, atol=2e-2)
# (B, M, N, w): windows that are multiples of 32 (whole-line column groups) and of 4 only (16-byte groups)
SHAPES = [(3, 1000, 64, 64), (2, 777, 128, 32), (2, 300, 64, 96), (5, 129, 128, 64), (3, 50, 64, 32), (1, 1, 64, 32),
          (2, 515, 128, 160), (3, 1000, 64, 100), (2, 777, 128, 36), (5, 515, 64, 8), (3, 301, 64, 44), (2, 64, 128, 12),
          (2, 2049, 64, 1024), (1, 700, 64, 128),
          # other head widths; windows that are not a multiple of 4 (band rows at 4-byte alignment only)
          (2, 777, 128, 33), (5, 1000, 32, 255), (2, 300, 96, 97), (9, 129, 16, 64), (3, 50, 48, 35), (2, 1030, 80, 513),
          (3, 333, 112, 161), (3, 515, 64, 41), (2, 200, 32, 100), (1, 4097, 96, 70)]


def bits(t):
    return t.contiguous().view(torch.int16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bfloat16", "float16"])
@pytest.mark.parametrize("B,M,N,w", SHAPES, ids=[f"B{B}-M{M}-N{N}-w{w}" for B, M, N, w in SHAPES])
def test_both_implementations_and_oracle(device, B, M, N, w, dtype):
    print(f"case B{B} M{M} N{N} w{w} {dtype}", flush=True)
    q, k, v, go = (seeded((B, M, N), 300 + s, dtype) for s in range(4))
    a, ga = (seeded((B, M, 2 * w + 1), 310 + s, dtype, 0.25) for s in range(2))
    # entries of an input band outside the sequence must never be read as numbers
    outside = ~oracle.band_mask(M, w, torch.device("cpu"))
    a[:, outside] = float("nan")
    ga[:, outside] = float("nan")
    dq, dk, dv, dgo, da, dga = (t.to(device) for t in (q, k, v, go, a, ga))
    kt = dk.transpose(1, 2)
    res = []
    for flags in (0, abi.NO_LDS_DIRECT):
        att = abi.window_forward(dq, kt, w, flags)
        out = abi.unwindow_forward(da, dv, w, flags)
        g_a, g_v = abi.unwindow_backward(da, dv, w, dgo, flags)
        g_q, g_k = abi.window_backward(dq, kt, w, dga, flags)
        res.append(dict(window_fwd=att, unwindow_fwd=out, grad_a=g_a, grad_v=g_v, grad_q=g_q, grad_k=g_k))
    for name in res[0]:
        torch.testing.assert_close(res[0][name].float(), res[1][name].float(), **TOL, msg=lambda m: f"{name}: {m}")
    for name in ("window_fwd", "grad_a") + (("unwindow_fwd", "grad_q") if w % 4 == 0 else ()):
        assert torch.equal(bits(res[0][name]), bits(res[1][name])), f"{name}: the two implementations sum in the same order"
    if B * M * (2 * w + 1) <= 2_500_000:  # the oracle's loops finish in seconds
        f = lambda t: t.float()  # noqa: E731
        a0, ga0 = a.clone(), ga.clone()
        a0[:, outside] = 0
        ga0[:, outside] = 0
        ktc = f(k).transpose(1, 2).contiguous()
        want_a, want_v = oracle.unwindow_matmul_backward(f(a0), f(v), w, f(go))
        want_q, want_k = oracle.window_matmul_backward(f(q), ktc, w, f(ga0))
        want = dict(window_fwd=oracle.window_matmul_forward(f(q), ktc, w), unwindow_fwd=oracle.unwindow_matmul_forward(f(a0), f(v), w),
                    grad_a=want_a, grad_v=want_v, grad_q=want_q, grad_k=want_k)
        for name in want:
            torch.testing.assert_close(res[0][name].cpu().float(), want[name], **TOL, msg=lambda m: f"{name} vs oracle: {m}")


@pytest.mark.parametrize("w", [32, 44])
def test_padded_operands(device, w):
    """Rows of v / grad_o / q padded to a longer stride, batch elements of the band padded so that they
    start at every 16-byte position of a 128-byte line, results written into padded tensors."""
    B, M, N, dtype = 4, 333, 64, torch.bfloat16
    W = 2 * w + 1
    pad_rows = lambda t: torch.cat([t, torch.full_like(t, float("nan"))], -1)[..., :N]  # noqa: E731  row stride 2N
    v, go = (seeded((B, M, N), 320 + s, dtype).to(device) for s in range(2))
    band_store = torch.full((B, M * W + 24), float("nan"), dtype=dtype, device=device)  # batch stride not a multiple of 64
    a = band_store[:, :M * W].view(B, M, W)
    a.copy_(seeded((B, M, W), 330, dtype, 0.25))
    vp, gop = pad_rows(v), pad_rows(go)
    assert vp.stride(1) == 2 * N and a.stride(0) == M * W + 24
    for flags in (abi.NO_LDS_DIRECT, 0):
        out = abi.unwindow_forward(a, vp, w, flags)
        _, g_v = abi.unwindow_backward(a, vp, w, gop, flags, want_a=False)
        if flags:
            want_out, want_gv = out, g_v
    assert torch.equal(bits(out), bits(want_out))
    torch.testing.assert_close(g_v.float(), want_gv.float(), **TOL)
    ref_out = abi.unwindow_forward(a.contiguous(), v, w, abi.FORCE_STRIDED)
    torch.testing.assert_close(out.float(), ref_out.float(), **TOL)


def test_kernel_choice_is_unchanged_by_the_switch(device):
    """Both implementations belong to the wide-band family: wm_kernel_choice names the family."""
    for op in (1, 2, 3):
        for flags in (0, abi.NO_LDS_DIRECT):
            assert abi.lib().wm_kernel_choice(op, 8, 4096, 128, 64, abi.DTYPES[torch.bfloat16], 1, flags).decode() == f"mfma_p{op}"


@pytest.mark.parametrize("B,M,N,w,dtype", [(26, 4099, 64, 580, torch.bfloat16), (7, 16390, 128, 516, torch.float16),
                                           (44, 8200, 32, 172, torch.bfloat16), (56, 4099, 64, 255, torch.bfloat16),
                                           (56, 4100, 64, 258, torch.float16), (7, 8200, 48, 1023, torch.bfloat16)],
                         ids=["N64-w580", "N128-w516", "N32-w172", "N64-w255", "N64-w258", "N48-w1023"])
def test_band_out_ring_of_lines(device, B, M, N, w, dtype):
    """A band beyond 220 MB whose rows do not begin a whole number of lines apart (w % 32 != 0) is
    written through a ring of two chunks per row, every row in whole lines of its own grid (16-byte
    pieces of the ring when w % 4 == 0, 4-byte units otherwise).  Every band entry is one dot product in a fixed order, so the result must equal, bit for
    bit, that of the kernel for unaligned bands (WM_FLAG_NO_ALIGNED_BAND: 16-byte stores on a common
    column grid), entries outside the sequence must be +0.0, and rows picked across the tensor must
    match the CPU oracle.  The band lives at three different offsets inside a poisoned buffer: nothing
    outside it may be written."""
    print(f"case B{B} M{M} N{N} w{w}", flush=True)
    W = 2 * w + 1
    assert B * M * W * 2 >= 220 << 20 and w % 32 != 0
    q, k = (seeded((B, M, N), 340 + s, dtype).to(device) for s in range(2))
    kt = k.transpose(1, 2)
    want = abi.window_forward(q, kt, w, abi.NO_ALIGNED_BAND)
    store = torch.empty(B * M * W + 128, dtype=dtype, device=device)
    for off in (0, 8, 40) if w % 4 == 0 else (0, 2, 38):
        store.fill_(float("nan"))
        band = store[off:off + B * M * W].view(B, M, W)
        got = abi.window_forward(q, kt, w, 0, out=band)
        assert torch.equal(bits(got), bits(want)), f"offset {off}"
        assert bool(torch.isnan(store[:off]).all()) and bool(torch.isnan(store[off + B * M * W:]).all()), f"offset {off}: wrote outside the band"
    outside = ~oracle.band_mask(M, w, device)
    assert not bits(want)[:, outside].any(), "band entries outside the sequence are not +0.0"
    # rows at the ends and in the middle of a few batch elements against the oracle (float32 of the rounded inputs)
    for b in (0, B - 1):
        for i0 in (0, M // 2 - 3, M - 40):
            rows = slice(i0, i0 + 40)
            lo, hi = max(i0 - w, 0), min(i0 + 40 + w, M)
            qs = torch.zeros(1, hi - lo, N)
            qs[0, i0 - lo:i0 - lo + 40] = q[b, rows].float().cpu()
            ks = k[b, lo:hi].float().cpu().unsqueeze(0)
            ref = oracle.window_matmul_forward(qs, ks.transpose(1, 2).contiguous(), w)[0, i0 - lo:i0 - lo + 40]
            torch.testing.assert_close(want[b, rows].float().cpu(), ref, **TOL)


@pytest.mark.parametrize("w", [16, 24, 40, 41, 64])
def test_band_at_an_odd_element_offset(device, w):
    """A band whose first element sits at an odd element offset is only 2-byte aligned: neither the
    16-byte pieces of the LDS-direct kernels nor the whole-line stores apply, the products take the
    kernels for unaligned bands (at w = 16 and 24 the narrow-band ones, which leave those windows
    to the LDS-direct kernels only for layouts those accept) and give the numbers of the aligned call."""
    B, M, N, dtype = 3, 700, 64, torch.bfloat16
    W = 2 * w + 1
    q, k, v, go = (seeded((B, M, N), 350 + s, dtype).to(device) for s in range(4))
    a = seeded((B, M, W), 360, dtype, 0.25).to(device)
    store = torch.full((B * M * W + 8,), float("nan"), dtype=dtype, device=device)
    odd = store[1:1 + B * M * W].view(B, M, W)
    assert odd.data_ptr() % 4 == 2
    want_att = abi.window_forward(q, k.transpose(1, 2), w)
    got_att = abi.window_forward(q, k.transpose(1, 2), w, out=odd)
    assert torch.equal(bits(got_att), bits(want_att)) and bool(torch.isnan(store[0])) and bool(torch.isnan(store[1 + B * M * W:]).all())
    odd.copy_(a)
    torch.testing.assert_close(abi.unwindow_forward(odd, v, w).float(), abi.unwindow_forward(a, v, w).float(), **TOL)
    g_a, g_v = abi.unwindow_backward(odd, v, w, go)
    w_a, w_v = abi.unwindow_backward(a, v, w, go)
    assert torch.equal(bits(g_a), bits(w_a))
    torch.testing.assert_close(g_v.float(), w_v.float(), **TOL)
    g_q, g_k = abi.window_backward(q, k.transpose(1, 2), w, odd)
    w_q, w_k = abi.window_backward(q, k.transpose(1, 2), w, a)
    torch.testing.assert_close(g_q.float(), w_q.float(), **TOL)
    torch.testing.assert_close(g_k.float(), w_k.float(), **TOL)
