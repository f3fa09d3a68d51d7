"""Seeded random shapes: the tuned kernel families against the untuned one, on the GPU.

The parity tests proper compare against the CPU oracle at hand-picked shapes.  This file adds
breadth: shapes, dtypes and windows drawn from a fixed seed, the library's own kernel choice
(narrow-band, wide-band MFMA, float32 MFMA) against the strided family, which shares no tiling,
staging or masking code with them and is itself checked against the oracle in
``test_gpu_parity.py``; and the fused attention kernels against the chain of the separate ops in
float32.  Tolerances as everywhere, per element: float32 rtol = atol = 1e-3, 16-bit rtol = atol = 2e-2;
band entries outside the sequence must be +0.0 on bits.  The float32 kernel families are also
compared with the CPU oracle directly, one shape each.
"""
import random

import pytest
import torch

import oracle
import wm_ctypes as abi

pytestmark = pytest.mark.gpu

B_SET = [1, 2, 3, 5, 9]
M_SET = [1, 7, 31, 64, 100, 128, 129, 255, 300, 513, 1000, 1500]
W_SET = [1, 2, 3, 4, 5, 8, 9, 12, 16, 17, 24, 32, 33, 40, 64, 100, 128, 200, 256, 700]


def _draw(seed, n, n_set, dtypes):
    rng = random.Random(seed)
    return [(rng.choice(dtypes), rng.choice(B_SET), rng.choice(M_SET), rng.choice(n_set), rng.choice(W_SET))
            for _ in range(n)]


def _randn(shape, g, dtype, dev, scale=1.0):
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(dev)


def _assert_close(got, want, tol, what):
    got, want = got.float(), want.float()
    assert torch.isfinite(got).all(), what
    torch.testing.assert_close(got, want, rtol=tol, atol=tol, msg=lambda m: f"{what}: {m}")


def _assert_close_in_scale(got, want, tol, what):
    """For the fused attention against a float32 chain: the fused backward starts from the output as
    stored (rounded to 16 bits), whose rounding enters every gradient through D = sum dO * O, so an
    element near zero can be off by tol times the scale of the tensor rather than of itself."""
    got, want = got.float(), want.float()
    assert torch.isfinite(got).all(), what
    if got.numel():
        scale = max(1.0, want.abs().max().item())
        torch.testing.assert_close(got, want, rtol=tol, atol=tol * scale, msg=lambda m: f"{what}: {m}")


def _assert_band_zeros(band, M, w, what):
    outside = band[:, ~oracle.band_mask(M, w, band.device)]
    ints = {2: torch.int16, 4: torch.int32}[outside.element_size()]
    assert not outside.view(ints).any(), f"{what}: a band entry outside the sequence is not +0.0"


MATMUL_CASES = _draw(1, 60, [8, 16, 24, 32, 48, 64, 80, 96, 112, 128],
                     [torch.bfloat16, torch.float16, torch.float32])


@pytest.mark.parametrize("dtype,B,M,N,w", MATMUL_CASES,
                         ids=[f"{str(d)[6:]}-B{B}-M{M}-N{N}-w{w}" for d, B, M, N, w in MATMUL_CASES])
def test_kernel_choice_agrees_with_strided_family(device, dtype, B, M, N, w):
    g = torch.Generator().manual_seed(B * 1000003 + M * 1009 + N * 31 + w)
    q, k, v, go = (_randn((B, M, N), g, dtype, device) for _ in range(4))
    a = _randn((B, M, 2 * w + 1), g, dtype, device, 0.2)
    kt = k.transpose(1, 2)
    tol = 1e-3 if dtype == torch.float32 else 2e-2
    results = []
    for flags in (0, abi.FORCE_STRIDED):
        att = abi.window_forward(q, kt, w, flags)
        out = abi.unwindow_forward(a, v, w, flags)
        ga, gv = abi.unwindow_backward(a, v, w, go, flags)
        gq, gk = abi.window_backward(q, kt, w, a, flags)
        results.append(dict(window_fwd=att, unwindow_fwd=out, grad_a=ga, grad_v=gv, grad_q=gq, grad_k=gk))
    for name in results[0]:
        _assert_close(results[0][name], results[1][name], tol, name)


@pytest.mark.parametrize("w", range(1, 33))
@pytest.mark.parametrize("dtype,B,M,N", [(torch.bfloat16, 3, 300, 64), (torch.float16, 2, 129, 16),
                                         (torch.bfloat16, 5, 1000, 128), (torch.float16, 2, 31, 96),
                                         (torch.float32, 3, 300, 64), (torch.float32, 2, 129, 48),
                                         (torch.float32, 5, 1000, 16), (torch.float32, 2, 65, 32)])
def test_every_narrow_window(device, dtype, B, M, N, w):
    """The band-in kernels lay their LDS image out differently for w % 4 == 0 and for the other
    windows, and the batch stride M (2w + 1) moves the band rows through every alignment; the
    float32 shapes are the ones the narrow-band float32 kernels take (N a multiple of 16 up to 64)."""
    g = torch.Generator().manual_seed(w * 131 + M)
    q, k, v, go = (_randn((B, M, N), g, dtype, device) for _ in range(4))
    a = _randn((B, M, 2 * w + 1), g, dtype, device, 0.2)
    results = []
    for flags in (0, abi.FORCE_STRIDED):
        att = abi.window_forward(q, k.transpose(1, 2), w, flags)
        out = abi.unwindow_forward(a, v, w, flags)
        ga, gv = abi.unwindow_backward(a, v, w, go, flags)
        gq, gk = abi.window_backward(q, k.transpose(1, 2), w, a, flags)
        results.append(dict(window_fwd=att, unwindow_fwd=out, grad_a=ga, grad_v=gv, grad_q=gq, grad_k=gk))
    for name in results[0]:
        _assert_close(results[0][name], results[1][name], 1e-3 if dtype == torch.float32 else 2e-2, name)
    for name in ("window_fwd", "grad_a"):
        _assert_band_zeros(results[0][name], M, w, name)


# one shape per float32 kernel family, against the CPU oracle itself (kernel_choice names the family)
F32_FAMILIES = [("vector_p2", 3, 300, 80, 4), ("narrow_p2", 2, 333, 64, 16), ("f32_mfma_p2", 2, 400, 80, 15),
                ("narrow_p1", 3, 257, 48, 24), ("f32_mfma_p1", 1, 515, 128, 15), ("vector_p3", 2, 129, 24, 9),
                ("f32_split_p2", 2, 400, 80, 64), ("f32_split_p1", 1, 515, 128, 100), ("f32_split_p3", 2, 300, 32, 40),
                ("f32_mfma_p2", 2, 300, 32, 40), ("f32_split_p1", 2, 260, 24, 130), ("f32_split_p3", 1, 700, 72, 350)]


@pytest.mark.parametrize("family,B,M,N,w", F32_FAMILIES, ids=[f"{f[0]}-N{f[3]}-w{f[4]}" for f in F32_FAMILIES])
def test_float32_families_match_the_oracle(device, family, B, M, N, w):
    op = int(family[-1])
    assert abi.lib().wm_kernel_choice(op, B, M, N, w, abi.DTYPES[torch.float32], 1, 0).decode() == family
    g = torch.Generator().manual_seed(N * 1000 + w)
    q, k, v, go = (torch.randn(B, M, N, generator=g) for _ in range(4))
    a = torch.randn(B, M, 2 * w + 1, generator=g) * 0.2
    dq, dk, dv, dgo, da = (t.to(device) for t in (q, k, v, go, a))
    kt = k.transpose(1, 2).contiguous()
    tol = dict(rtol=1e-3, atol=1e-3)
    att = abi.window_forward(dq, dk.transpose(1, 2), w)
    torch.testing.assert_close(att.cpu(), oracle.window_matmul_forward(q, kt, w), **tol)
    _assert_band_zeros(att, M, w, "window_fwd")
    torch.testing.assert_close(abi.unwindow_forward(da, dv, w).cpu(), oracle.unwindow_matmul_forward(a, v, w), **tol)
    ga, gv = abi.unwindow_backward(da, dv, w, dgo)
    wa, wv = oracle.unwindow_matmul_backward(a, v, w, go)
    torch.testing.assert_close(ga.cpu(), wa, **tol)
    torch.testing.assert_close(gv.cpu(), wv, **tol)
    gq, gk = abi.window_backward(dq, dk.transpose(1, 2), w, da)
    wq, wk = oracle.window_matmul_backward(q, kt, w, a)
    torch.testing.assert_close(gq.cpu(), wq, **tol)
    torch.testing.assert_close(gk.cpu(), wk, **tol)


ATTENTION_CASES = _draw(2, 40, [16, 32, 48, 64, 80, 96, 112, 128], [torch.bfloat16, torch.float16])


@pytest.mark.parametrize("dtype,B,M,N,w", ATTENTION_CASES,
                         ids=[f"{str(d)[6:]}-B{B}-M{M}-N{N}-w{w}" for d, B, M, N, w in ATTENTION_CASES])
def test_fused_attention_agrees_with_chain_of_ops(device, dtype, B, M, N, w):
    rng = random.Random(B * 7919 + M * 104729 + N * 13 + w)
    mask = rng.choice([False, True])
    scale = rng.choice([1.0, 2.0]) / N ** 0.5  # the usual 1 / sqrt(N), and scores twice as wide
    g = torch.Generator().manual_seed(rng.randrange(1 << 30))
    q, k, v, go = (_randn((B, M, N), g, dtype, device) for _ in range(4))
    o, lse = abi.attention_forward(q, k, v, w, scale, mask)
    gq, gk, gv = abi.attention_backward(q, k, v, o, lse, go, w, scale)
    # the same chain on float32 copies of the rounded inputs
    qf, kf, vf, gof = (t.float() for t in (q, k, v, go))
    p = abi.band_softmax_forward(abi.window_forward(qf, kf.transpose(1, 2), w), scale, mask)
    _assert_close_in_scale(o, abi.unwindow_forward(p, vf, w), 2e-2, "output")
    gp, gv_ref = abi.unwindow_backward(p, vf, w, gof)
    gq_ref, gk_ref = abi.window_backward(qf, kf.transpose(1, 2), w, abi.band_softmax_backward(p, gp, scale, mask))
    _assert_close_in_scale(gq, gq_ref, 2e-2, "grad_q")
    _assert_close_in_scale(gk, gk_ref.transpose(1, 2), 2e-2, "grad_k")
    _assert_close_in_scale(gv, gv_ref, 2e-2, "grad_v")


@pytest.mark.parametrize("B,M,N,w", [(2, 700, 80, 300), (1, 515, 128, 100), (2, 300, 32, 40), (3, 200, 8, 16), (1, 1100, 64, 1200)])
def test_split_float32_kernels_keep_float32_accuracy(device, B, M, N, w):
    """The float32 products that run on the bf16 matrix instruction (every value cut into three bf16
    parts, six of the nine partial products kept) against the dense float64 formulation: their largest
    error may be no more than four times that of the kernels on the float32 matrix instruction
    (WM_FLAG_NO_SPLIT_F32) on the same inputs, i.e. rounding noise of float32 accumulation, nothing
    that scales with the 2^-8 of a bf16 operand or the 2^-16 of a two-part split."""
    g = torch.Generator().manual_seed(7 * N + w)
    q, k, v, go = (torch.randn(B, M, N, generator=g) * 3.0 for _ in range(4))
    a, ga = (torch.randn(B, M, 2 * w + 1, generator=g) for _ in range(2))
    kt = k.transpose(1, 2).contiguous()
    want = dict(att=oracle.dense_window_matmul(q, kt, w), out=oracle.dense_unwindow_matmul(a, v, w))
    want["grad_a"], want["grad_v"] = oracle.dense_unwindow_matmul_backward(a, v, w, go)
    want["grad_q"], gkt = oracle.dense_window_matmul_backward(q, kt, w, ga)
    want["grad_k"] = gkt.transpose(1, 2)
    dq, dk, dv, dgo, da, dga = (t.to(device) for t in (q, k, v, go, a, ga))
    worst = {}
    for flags in (0, abi.NO_SPLIT_F32):
        got = dict(att=abi.window_forward(dq, dk.transpose(1, 2), w, flags), out=abi.unwindow_forward(da, dv, w, flags))
        got["grad_a"], got["grad_v"] = abi.unwindow_backward(da, dv, w, dgo, flags)
        got["grad_q"], gk = abi.window_backward(dq, dk.transpose(1, 2), w, dga, flags)
        got["grad_k"] = gk.transpose(1, 2)  # the entry point returns grad_k in the (B, N, M) layout of k
        worst[flags] = {n: float((got[n].cpu().double() - want[n].double()).abs().max()) for n in want}
    for n in want:
        scale = float(want[n].double().abs().max())
        assert worst[0][n] <= 4 * worst[abi.NO_SPLIT_F32][n] + 1e-7 * scale, (n, worst[0][n], worst[abi.NO_SPLIT_F32][n])
        assert worst[0][n] <= 2e-5 * scale, (n, worst[0][n], scale)
