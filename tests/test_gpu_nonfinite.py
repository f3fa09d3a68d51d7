"""How far a non-finite value in a VALID operand row travels.

The reference's CPU path only ever multiplies rows that lie inside the window (reference
cpu/window_matmul_cpu.cpp:39-43, 129-141), so an Inf in row c of k, v, q or grad_o reaches the
outputs of rows |i - c| <= w and nothing else.  The matrix-instruction kernels (and the float64
tile kernels) multiply whole tiles in which entries outside the band are exact zeros, and 0 * Inf = NaN: there the value can
also reach rows of the same tile that are outside the window.  This file pins that behaviour as a
contract, against the CPU oracle run on the same poisoned inputs:

  * every output element that is non-finite in the oracle is non-finite on the GPU (nothing is lost);
  * rows farther than REACH(w) = w + 320 from the poisoned row are bit-identical to a run on clean
    inputs (the spread is bounded by one tile of at most 256 rows plus one 64-row chunk);
  * the strided kernels, which multiply in-window rows only like the reference, stay within w rows
    and their finite outputs equal the clean run bit for bit.
"""
import math

import pytest
import torch

import oracle
import wm_ctypes as abi
from conftest import seeded

pytestmark = pytest.mark.gpu

M, N, ROW = 2048, 64, 1000
WINDOWS = [3, 8, 24, 64, 256]
DTYPES = [torch.bfloat16, torch.float16, torch.float32, torch.float64]


def reach(w):
    return w + 320


def bits(t):
    return t.contiguous().view({2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()])


def rows_equal(a, b):
    """Per-row bitwise equality of two (1, M, X) tensors -> bool vector of length M."""
    return (bits(a) == bits(b)).all(dim=-1)[0].cpu()


def check(name, clean, dirty, want_dirty, w, flags):
    far = (torch.arange(M) - ROW).abs() > (w if flags == abi.FORCE_STRIDED else reach(w))
    same = rows_equal(clean, dirty)
    assert bool(same[far].all()), f"{name}: a row more than {reach(w)} rows from the poisoned one changed"
    lost = ~torch.isfinite(want_dirty) & torch.isfinite(dirty.cpu().to(want_dirty.dtype))
    assert not bool(lost.any()), f"{name}: a non-finite value of the reference result is finite here"
    if flags == abi.FORCE_STRIDED:
        fin = torch.isfinite(want_dirty)
        assert torch.equal(bits(dirty.cpu())[fin], bits(clean.cpu())[fin]), f"{name}: finite outputs moved"


@pytest.mark.parametrize("flags", [0, abi.FORCE_STRIDED], ids=["auto", "strided"])
@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("w", WINDOWS)
def test_one_poisoned_row_stays_local(device, w, dtype, flags):
    print(f"case w={w} {dtype} flags={flags}", flush=True)
    q, k, v, go = (seeded((1, M, N), 70 + s, dtype) for s in range(4))
    a, ga = (seeded((1, M, 2 * w + 1), 80 + s, dtype, 0.25) for s in range(2))

    def poisoned(t, value):
        t = t.clone()
        t[0, ROW, 5] = value
        return t

    dev = lambda *ts: [t.to(device) for t in ts]  # noqa: E731
    dq, dk, dv, dgo, da, dga = dev(q, k, v, go, a, ga)
    kt = lambda t: t.transpose(1, 2)  # noqa: E731
    inf, nan = float("inf"), float("nan")

    # window forward: Inf in a key row
    kp = poisoned(k, inf)
    check("window_forward / k", abi.window_forward(dq, kt(dk), w, flags), abi.window_forward(dq, kt(kp.to(device)), w, flags),
          oracle.window_matmul_forward(q.float(), kt(kp.float()).contiguous(), w), w, flags)
    # unwindow forward: NaN in a value row
    vp = poisoned(v, nan)
    check("unwindow_forward / v", abi.unwindow_forward(da, dv, w, flags), abi.unwindow_forward(da, vp.to(device), w, flags),
          oracle.unwindow_matmul_forward(a.float(), vp.float(), w), w, flags)
    # unwindow backward: Inf in an upstream gradient row reaches grad_a and grad_v
    gp = poisoned(go, -inf)
    cA, cV = abi.unwindow_backward(da, dv, w, dgo, flags)
    pA, pV = abi.unwindow_backward(da, dv, w, gp.to(device), flags)
    wA, wV = oracle.unwindow_matmul_backward(a.float(), v.float(), w, gp.float())
    check("unwindow_backward / grad_o -> grad_a", cA, pA, wA, w, flags)
    check("unwindow_backward / grad_o -> grad_v", cV, pV, wV, w, flags)
    # window backward: NaN in a query row reaches grad_k, Inf in a key row reaches grad_q
    qp = poisoned(q, nan)
    cQ, cK = abi.window_backward(dq, kt(dk), w, dga, flags)
    _, pK = abi.window_backward(qp.to(device), kt(dk), w, dga, flags, want_q=False)
    _, wK = oracle.window_matmul_backward(qp.float(), kt(k.float()).contiguous(), w, ga.float())
    check("window_backward / q -> grad_k", cK.transpose(1, 2), pK.transpose(1, 2), wK.transpose(1, 2), w, flags)
    pQ, _ = abi.window_backward(dq, kt(kp.to(device)), w, dga, flags, want_k=False)
    wQ, _ = oracle.window_matmul_backward(q.float(), kt(kp.float()).contiguous(), w, ga.float())
    check("window_backward / k -> grad_q", cQ, pQ, wQ, w, flags)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bfloat16", "float16"])
@pytest.mark.parametrize("w", [8, 64, 256])
def test_fused_attention_poisoned_value_row(device, w, dtype):
    """The fused kernels share the rule: a NaN value row reaches at most one tile beyond the window,
    and every output row inside the window of the poisoned key is non-finite as in the chain."""
    q, k, v = (seeded((1, M, N), 90 + s, dtype).to(device) for s in range(3))
    scale = 1.0 / math.sqrt(N)
    clean, _ = abi.attention_forward(q, k, v, w, scale)
    vp = v.clone()
    vp[0, ROW, 7] = float("nan")
    dirty, _ = abi.attention_forward(q, k, vp, w, scale)
    dist = (torch.arange(M) - ROW).abs()
    same = rows_equal(clean, dirty)
    assert bool(same[dist > reach(w)].all())
    assert bool(torch.isnan(dirty[0, :, 7].cpu().float())[dist <= w].all())


@pytest.mark.parametrize("which", ["v", "grad_o"])
@pytest.mark.parametrize("w", [8, 32, 64, 256])
def test_fused_attention_backward_poisoned_row(device, w, which):
    """The fused backward (one kernel up to w = 32 at this head width, two kernels above) under the same
    rule: a NaN in one row of v or of the upstream gradient changes no gradient row farther than
    REACH(w) from it, and the rows the chain would poison are non-finite here too."""
    dtype = torch.bfloat16
    q, k, v, go = (seeded((1, M, N), 95 + s, dtype).to(device) for s in range(4))
    scale = 1.0 / math.sqrt(N)
    o, lse = abi.attention_forward(q, k, v, w, scale)
    clean = abi.attention_backward(q, k, v, o, lse, go, w, scale)
    vp, gp = v.clone(), go.clone()
    (vp if which == "v" else gp)[0, ROW, 7] = float("nan")
    dirty = abi.attention_backward(q, k, vp, o, lse, gp, w, scale)
    dist = (torch.arange(M) - ROW).abs()
    for name, c, d in zip(("grad_q", "grad_k", "grad_v"), clean, dirty):
        same = rows_equal(c, d)
        assert bool(same[dist > reach(w)].all()), f"{name}: a row more than {reach(w)} rows from the poisoned one changed"
    gq, gk, gv = dirty
    if which == "v":
        # dP[i, ROW] = grad_o_i . v_ROW is NaN for every query i in the window of key ROW: grad_q_i and grad_k_ROW
        assert bool(torch.isnan(gq[0].float()).any(dim=-1).cpu()[dist <= w].all())
        assert bool(torch.isnan(gk[0, ROW].float()).any())
    else:
        # grad_v_c takes P[ROW, c] * grad_o_ROW for every key c in the window of query ROW
        assert bool(torch.isnan(gv[0, :, 7].float()).cpu()[dist <= w].all())
        assert bool(torch.isnan(gq[0, ROW].float()).any())
