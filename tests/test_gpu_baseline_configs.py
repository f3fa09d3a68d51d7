"""The BASELINE workloads at their full sizes on the GPU.

The CPU oracle cannot finish these in seconds, so each is checked three ways:
  * exactly-computed row blocks: for sampled (batch, row range) the expected band rows and
    outputs are formed with small dense float64 matmuls on the GPU (library routines only);
  * size-independent properties: row sums of the band against a cumulative-sum closed form
    (bounded by the rounding of the stored values themselves, so that one dropped band entry
    or one dropped value row fails), the adjoint identities between forward and backward,
    exact +0.0 outside the sequence, zero rows of q giving exact zero band rows;
  * the golden fixtures cover the same workloads at reduced size against the CPU oracle.
Tolerances: float32 1e-3, bfloat16 / float16 2e-2 (relative and absolute), as stated for the path.
"""
import pytest
import torch

import oracle
from conftest import seeded

pytestmark = pytest.mark.gpu


def band_rows_expected(q, k, w, b, r0, r1):
    """Rows r0..r1 of window_matmul(q, k^T) for batch b, float64, by a small dense product."""
    M = q.shape[1]
    c0, c1 = max(r0 - w, 0), min(r1 + w, M)
    S = q[b, r0:r1].double() @ k[b, c0:c1].double().T  # (rows, c1-c0)
    i = torch.arange(r0, r1, device=q.device).unsqueeze(1)
    j = torch.arange(2 * w + 1, device=q.device).unsqueeze(0)
    c = i + j - w
    valid = (c >= 0) & (c < M)
    gathered = torch.gather(S, 1, (c - c0).clamp(0, c1 - c0 - 1))
    return torch.where(valid, gathered, torch.zeros((), dtype=S.dtype, device=S.device))


def unwindow_rows_expected(a, v, w, b, r0, r1):
    M = v.shape[1]
    c0, c1 = max(r0 - w, 0), min(r1 + w, M)
    i = torch.arange(r0, r1, device=a.device).unsqueeze(1)
    j = torch.arange(2 * w + 1, device=a.device).unsqueeze(0)
    c = i + j - w
    valid = (c >= 0) & (c < M)
    D = torch.zeros(r1 - r0, c1 - c0, dtype=torch.float64, device=a.device)
    D.scatter_add_(1, (c - c0).clamp(0, c1 - c0 - 1), torch.where(valid, a[b, r0:r1].double(), torch.zeros((), dtype=torch.float64, device=a.device)))
    return D @ v[b, c0:c1].double()


def transposed_rows_expected(a, g, w, b, c0, c1):
    """Rows c0..c1 of P3(a, g): out[c] = sum_r a[r, c-r+w] g[r]."""
    M = g.shape[1]
    r0, r1 = max(c0 - w, 0), min(c1 + w, M)
    r = torch.arange(r0, r1, device=a.device).unsqueeze(1)
    c = torch.arange(c0, c1, device=a.device).unsqueeze(0)
    j = c - r + w
    valid = (j >= 0) & (j <= 2 * w)
    T = torch.gather(a[b, r0:r1].double(), 1, j.clamp(0, 2 * w))
    T = torch.where(valid, T, torch.zeros((), dtype=torch.float64, device=a.device))  # (rows r, cols c)
    return T.T @ g[b, r0:r1].double()


def window_sum(x, w):
    """out[b, i] = sum_{c in window(i)} x[b, c] in float64 via cumulative sums."""
    M = x.shape[1]
    cs = torch.cat([torch.zeros_like(x[:, :1]), x.cumsum(1)], 1)
    i = torch.arange(M, device=x.device)
    return cs[:, (i + w + 1).clamp(max=M)] - cs[:, (i - w).clamp(min=0)]


def check(got, want, tol, what):
    torch.testing.assert_close(got.double(), want, rtol=tol, atol=tol, msg=lambda s: f"{what}: {s}")


def storage_eps(dtype):
    """Largest relative error of rounding a float32 accumulator to `dtype` (float32 results are not
    rounded again; what differs from an exact sum there is the order of the float32 accumulation)."""
    return {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -24}[dtype]


def check_bounded(got, want, bound, what):
    excess = (got.double() - want).abs() - bound
    worst = float(excess.max())
    assert worst <= 0.0, f"{what}: error exceeds its rounding bound by {worst:.3e} (bound there {float(bound.flatten()[excess.argmax()]):.3e})"


def run_config(device, B, M, N, w, dtype, tol, qk_scale=1.0, backward=True, zero_rows=False, blocks=3, rows=192,
               uniform_band=False):
    from window_matmul import unwindow_matmul, window_matmul

    q = seeded((B, M, N), 11, dtype, qk_scale).to(device)
    k = seeded((B, M, N), 12, dtype, qk_scale).to(device)
    v = seeded((B, M, N), 13, dtype).to(device)
    go = seeded((B, M, N), 14, dtype).to(device)
    zr = None
    if zero_rows:
        g = torch.Generator().manual_seed(5)
        zr = torch.randperm(M, generator=g)[: M // 20].to(device)
        q[:, zr] = 0
    q.requires_grad_(backward), k.requires_grad_(backward), v.requires_grad_(backward)
    att = window_matmul(q, k.transpose(1, 2), w)
    mask = oracle.band_mask(M, w, device)
    if uniform_band:
        # the band the configuration names for unwindow_matmul: uniform[0, 1) per entry, rows normalised
        # to sum 1 (over all 2w+1 entries; those outside the sequence are never read)
        g = torch.Generator().manual_seed(16)
        probs = torch.empty(B, M, 2 * w + 1, dtype=dtype, device=device)
        for b in range(B):  # batch element by batch element: the float32 draw of the whole band would be 2 GiB
            u = torch.rand(M, 2 * w + 1, generator=g).to(device)
            probs[b] = (u / u.sum(-1, keepdim=True)).to(dtype)
        probs.requires_grad_(backward)
    else:
        probs = torch.softmax(att.float(), -1).to(dtype).detach().requires_grad_(backward)
    out = unwindow_matmul(probs, v, w)

    # exact zeros outside the sequence; zero q rows give exact zero band rows
    assert not att.detach()[:, ~mask].view(torch.int16 if att.element_size() == 2 else torch.int32).any()
    if zr is not None:
        assert not att.detach()[:, zr].view(torch.int16 if att.element_size() == 2 else torch.int32).any()

    # closed forms over the whole tensor: row sums of the band, and unwindow with a band of ones
    # Bounds from the stored values: each band entry is a float32 accumulation (error at most
    # N 2^-24 sum_h |q_h k_h|, taken as 4 N 2^-24 |q| . window_sum(|k|) over a row) rounded once to the
    # storage type (relative error eps, independent from entry to entry: 8 eps times the 2-norm of the
    # row is beyond ten standard deviations of their sum, and far below one typical entry).
    eps = storage_eps(dtype)
    ksum = window_sum(k.detach().double(), w)  # (B, M, N)
    kabs = window_sum(k.detach().double().abs(), w)
    a64 = att.detach().double()
    bound = 8 * eps * a64.pow(2).sum(-1).sqrt() + 4 * N * 2.0 ** -24 * (q.detach().double().abs() * kabs).sum(-1) + 1e-6
    check_bounded(a64.sum(-1), (q.detach().double() * ksum).sum(-1), bound, "band row sums")
    del a64, kabs, ksum
    ones = torch.ones(B, M, 2 * w + 1, dtype=dtype, device=device)
    ones[:, ~mask] = float("nan")  # must be ignored
    # one float32 accumulation of up to 2w+1 value rows, rounded once
    want = window_sum(v.detach().double(), w)
    bound = 2 * eps * want.abs() + 4 * (2 * w + 1) * 2.0 ** -24 * window_sum(v.detach().double().abs(), w) + 1e-6
    check_bounded(unwindow_matmul(ones, v.detach(), w), want, bound, "sliding sums")
    del ones, want, bound

    gA = gV = gQ = gK = None
    if backward:
        out.backward(go)
        gA, gV = probs.grad, v.grad
        ga_up = seeded((B, M, 2 * w + 1), 15, dtype, 0.25).to(device)
        att.backward(ga_up)
        gQ, gK = q.grad, k.grad
        assert not gA[:, ~mask].view(torch.int16 if gA.element_size() == 2 else torch.int32).any()
        # adjoint identities in float64 on the stored values
        lhs = (att.detach().double() * ga_up.double()).sum()
        scale = float(lhs.abs()) + float((att.detach().double().abs() * ga_up.double().abs()).sum()) * tol
        assert abs(float(lhs - (q.detach().double() * gQ.double()).sum())) <= tol * scale + 1e-6
        assert abs(float(lhs - (k.detach().double() * gK.double()).sum())) <= tol * scale + 1e-6

    # exactly-computed row blocks
    # per sampled batch element: both ends of the sequence, a block at a random offset, one that has a
    # seam between two 128-row tiles in its middle and one around a 64-row chunk seam that is not a tile seam
    gen = torch.Generator().manual_seed(3)
    for _ in range(blocks):
        b = int(torch.randint(B, (1,), generator=gen))
        r0 = int(torch.randint(max(M - rows, 1), (1,), generator=gen))
        tile = 128 * int(torch.randint(1, max(M // 128, 2), (1,), generator=gen))
        chunk = 128 * int(torch.randint(0, max(M // 128, 1), (1,), generator=gen)) + 64
        starts = {0, r0, max(M - rows, 0), min(max(tile - rows // 2, 0), max(M - rows, 0)),
                  min(max(chunk - rows // 2, 0), max(M - rows, 0))}
        for r0 in sorted(starts):
            r1 = min(r0 + rows, M)
            check(att.detach()[b, r0:r1], band_rows_expected(q.detach(), k.detach(), w, b, r0, r1), tol, "window fwd")
            check(out.detach()[b, r0:r1], unwindow_rows_expected(probs.detach(), v.detach(), w, b, r0, r1), tol, "unwindow fwd")
            if backward:
                check(gA[b, r0:r1], band_rows_expected(go, v.detach(), w, b, r0, r1), tol, "grad_a")
                check(gV[b, r0:r1], transposed_rows_expected(probs.detach(), go, w, b, r0, r1), tol, "grad_v")
                check(gQ[b, r0:r1], unwindow_rows_expected(ga_up, k.detach(), w, b, r0, r1), tol, "grad_q")
                check(gK[b, r0:r1], transposed_rows_expected(ga_up, q.detach(), w, b, r0, r1), tol, "grad_k")


def test_config2_small_window_bf16(device):
    run_config(device, B=96, M=16384, N=64, w=8, dtype=torch.bfloat16, tol=2e-2, backward=False)


def test_config3_local_attention_bf16(device):
    run_config(device, B=96, M=4096, N=64, w=256, dtype=torch.bfloat16, tol=2e-2, qk_scale=0.125, blocks=6)


def test_config4_wide_head_fp16(device):
    run_config(device, B=16, M=32768, N=128, w=512, dtype=torch.float16, tol=2e-2, blocks=4, uniform_band=True)


@pytest.mark.parametrize("w", [1, 33, 1500])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-3), (torch.bfloat16, 2e-2)], ids=["f32", "bf16"])
def test_config5_ragged(device, w, dtype, tol):
    run_config(device, B=7, M=3001, N=80, w=w, dtype=dtype, tol=tol, zero_rows=True, blocks=2, rows=150)


def test_config1_plumbing_contiguous_keys(device):
    """BASELINE config 1 states k as a contiguous (2, 64, 128) tensor."""
    from window_matmul import unwindow_matmul, window_matmul

    B, M, N, w = 2, 128, 64, 4
    q = seeded((B, M, N), 1).to(device).requires_grad_(True)
    kt = seeded((B, N, M), 2).to(device).requires_grad_(True)
    v = seeded((B, M, N), 3).to(device).requires_grad_(True)
    go = seeded((B, M, N), 4).to(device)
    att = window_matmul(q, kt, w)
    out = unwindow_matmul(att, v, w)
    out.backward(go)
    ra = oracle.dense_window_matmul(q.detach(), kt.detach(), w)
    ro = oracle.dense_unwindow_matmul(ra, v.detach(), w)
    rga, rgv = oracle.dense_unwindow_matmul_backward(ra, v.detach(), w, go)
    rgq, rgkt = oracle.dense_window_matmul_backward(q.detach(), kt.detach(), w, rga)
    for got, want in ((att, ra), (out, ro), (v.grad, rgv), (q.grad, rgq), (kt.grad, rgkt)):
        torch.testing.assert_close(got.detach().double(), want, rtol=1e-3, atol=1e-3)
    assert kt.grad.shape == (B, N, M)
