"""GPU tests of the drop-in Python API (window_matmul.window_matmul / unwindow_matmul and
their autograd Functions), in the manner of the reference's own tests: the custom op
against an independent torch formulation, outputs and input gradients
(reference tests/test_window_matmul.py:53-84, tests/test_unwindow_matmul.py:40-79,
tests/test_attention.py:90-140)."""
import ctypes
import itertools
import math

import pytest
import torch

import oracle
from conftest import seeded

pytestmark = pytest.mark.gpu

DIMS = [(2, 1, 1, 3), (2, 1, 4, 3), (2, 1, 16, 3), (2, 1, 32, 3), (2, 1, 16, 32), (2, 3, 77, 16)]  # (batch, heads, M, N)
WINDOWS = [0, 1, 4, 16]


def head_major(batch, heads, M, N, seed, device, dtype=torch.float32):
    """randn(batch, M, heads*N) viewed as (batch, heads, M, N): non-contiguous (reference tests/utils.py:38-44)."""
    t = seeded((batch, M, heads * N), seed, dtype).to(device)
    return t.view(batch, M, heads, N).transpose(1, 2)


def dense_window(q, kt, w):
    if not w:
        return (q * kt.transpose(-1, -2)).sum(-1, keepdim=True)
    lead = q.shape[:-2]
    S = torch.matmul(q, kt).reshape(-1, q.shape[-2], q.shape[-2])
    return oracle.dense_to_band(S, w).reshape(*lead, q.shape[-2], 2 * w + 1)


def dense_unwindow(a, v, w):
    if not w:
        return a * v
    lead = v.shape[:-2]
    D = oracle.band_to_dense(a.reshape(-1, a.shape[-2], a.shape[-1]), w).reshape(*lead, v.shape[-2], v.shape[-2])
    return torch.matmul(D, v)


@pytest.mark.parametrize("dim", DIMS)
@pytest.mark.parametrize("w", WINDOWS)
def test_window_matmul_forward_and_grads(device, dim, w):
    from window_matmul import window_matmul

    q0 = head_major(*dim, 1, device)
    k0 = head_major(*dim, 2, device)
    res = {}
    for name, fn in (("dense", dense_window), ("custom", window_matmul)):
        q = q0.detach().clone().requires_grad_(True)
        k = k0.detach().clone().requires_grad_(True)
        att = fn(q, k.transpose(-1, -2), w)
        # arange-weighted loss gives a known, non-uniform upstream gradient (reference tests/test_window_matmul.py:71)
        (att * torch.arange(att.numel(), device=device).to(att).view_as(att)).mean().backward()
        res[name] = (att, q.grad, k.grad)
    assert res["custom"][0].shape == (*dim[:3], 2 * w + 1)
    for x, y in zip(res["custom"], res["dense"]):
        torch.testing.assert_close(x, y, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dim", DIMS)
@pytest.mark.parametrize("w", WINDOWS)
def test_unwindow_matmul_forward_and_grads(device, dim, w):
    from window_matmul import unwindow_matmul

    batch, heads, M, N = dim
    a0 = seeded((batch, heads, M, 2 * w + 1), 3, torch.float32).to(device)
    v0 = head_major(*dim, 4, device)
    res = {}
    for name, fn in (("dense", dense_unwindow), ("custom", unwindow_matmul)):
        a = a0.detach().clone().requires_grad_(True)
        v = v0.detach().clone().requires_grad_(True)
        out = fn(a, v, w)
        (out * torch.arange(out.numel(), device=device).to(out).view_as(out)).mean().backward()
        ga = a.grad
        if w:
            mask = oracle.band_mask(M, w, device)
            # the dense formulation propagates no gradient to invalid entries; ours writes +0.0 there
            assert torch.equal(ga[..., ~mask], torch.zeros_like(ga[..., ~mask]))
        res[name] = (out, ga, v.grad)
    for x, y in zip(res["custom"], res["dense"]):
        torch.testing.assert_close(x, y, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dim", DIMS[:5])
def test_window_size_zero_on_gpu(device, dim):
    from window_matmul import unwindow_matmul, window_matmul

    q, k, v = (head_major(*dim, s, device) for s in (1, 2, 3))
    att = window_matmul(q, k.transpose(-1, -2), 0)
    out = unwindow_matmul(att.softmax(-1), v, 0)
    assert att.shape[-1] == 1
    assert torch.allclose(out, v)  # reference tests/test_attention.py:86-87


class Layer(torch.nn.Module):
    """window -> /sqrt(N) -> softmax over the whole band -> unwindow -> linear -> sigmoid
    (the caller the reference tests, tests/test_attention.py:48-72)."""

    def __init__(self, w, fns, linear):
        super().__init__()
        self.w, self.fns, self.linear = w, fns, linear

    def forward(self, q, k, v):
        win, unwin = self.fns
        p = torch.softmax(win(q, k.transpose(-1, -2), self.w) / math.sqrt(q.shape[-1]), dim=-1)
        return torch.sigmoid(self.linear(unwin(p, v, self.w)))


@pytest.mark.parametrize("dim", DIMS)
@pytest.mark.parametrize("w", WINDOWS)
def test_three_layer_attention_chain(device, dim, w):
    from window_matmul import unwindow_matmul, window_matmul

    torch.manual_seed(0)
    linear = torch.nn.Linear(dim[-1], dim[-1]).to(device)
    res = {}
    for name, fns in (("dense", (dense_window, dense_unwindow)), ("custom", (window_matmul, unwindow_matmul))):
        q, k, v = (head_major(*dim, s, device).detach().clone().requires_grad_(True) for s in (1, 2, 3))
        x = (q, k, v)
        for _ in range(3):
            out = Layer(w, fns, linear)(*x)
            x = (linear(out), linear(out), linear(out))
        out.mean().backward()
        res[name] = (out, q.grad, k.grad, v.grad)
    for x, y in zip(res["custom"], res["dense"]):
        torch.testing.assert_close(x, y, rtol=1e-4, atol=1e-5)


def test_gradcheck_float64(device):
    from window_matmul import unwindow_matmul, window_matmul

    B, M, N, w = 2, 7, 3, 2
    q = seeded((B, M, N), 1, torch.float64).to(device).requires_grad_(True)
    kt = seeded((B, N, M), 2, torch.float64).to(device).requires_grad_(True)
    v = seeded((B, M, N), 3, torch.float64).to(device).requires_grad_(True)
    mask = oracle.band_mask(M, w, device)
    a = (seeded((B, M, 2 * w + 1), 4, torch.float64).to(device) * mask).requires_grad_(True)
    assert torch.autograd.gradcheck(lambda x, y: window_matmul(x, y, w), (q, kt))
    # invalid band entries carry no dependence; restrict the check to valid ones
    assert torch.autograd.gradcheck(lambda x, y: unwindow_matmul(x * mask, y, w), (a, v))


def test_autocast_casts_to_float16(device):
    """Under autocast the Functions run in float16 (reference window_matmul.py:9,45)."""
    from window_matmul import unwindow_matmul, window_matmul

    B, M, N, w = 2, 40, 16, 4
    q, k, v = (seeded((B, M, N), s).to(device) for s in (1, 2, 3))
    with torch.autocast("cuda", dtype=torch.bfloat16):
        att = window_matmul(q, k.transpose(1, 2), w)
        out = unwindow_matmul(att.float().softmax(-1), v, w)
    assert att.dtype == torch.float16 and out.dtype == torch.float16
    want = oracle.dense_window_matmul(q.half().cpu(), k.half().cpu().transpose(1, 2), w)
    torch.testing.assert_close(att.cpu().double(), want, rtol=2e-2, atol=2e-2)


def test_error_behaviour(device):
    import window_matmul_kernel as native

    q = torch.zeros(2, 8, 4, device=device)
    with pytest.raises(RuntimeError, match="Input mismatch"):
        native.window_matmul_forward(q, torch.zeros(2, 8, 4, device=device), 1)
    with pytest.raises(RuntimeError, match="Input mismatch"):
        native.unwindow_matmul_forward(torch.zeros(2, 8, 4, device=device), q, 1)
    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        native.window_matmul_forward(q, torch.zeros(2, 4, 8), 1)
    with pytest.raises(RuntimeError, match="not implemented for"):
        native.window_matmul_forward(q.int(), torch.zeros(2, 4, 8, device=device).int(), 1)


@pytest.mark.parametrize("which", ["first", "second"])
def test_gradient_of_one_input_only(device, which):
    """Only the requested gradient is produced, and it equals the one of the two-sided backward."""
    import window_matmul_kernel as native
    from window_matmul import unwindow_matmul, window_matmul

    B, M, N, w = 3, 96, 32, 12
    q0, k0, v0 = (seeded((B, M, N), s, torch.float32).to(device) for s in (31, 32, 33))
    a0 = seeded((B, M, 2 * w + 1), 34, torch.float32).to(device)
    first = which == "first"

    q = q0.clone().requires_grad_(first)
    k = k0.clone().requires_grad_(not first)
    window_matmul(q, k.transpose(-1, -2), w).square().sum().backward()
    att = native.window_matmul_forward(q0, k0.transpose(-1, -2), w)
    gq, gk = native.window_matmul_backward(q0, k0.transpose(-1, -2), w, 2 * att)
    torch.testing.assert_close(q.grad if first else k.grad, gq if first else gk.transpose(-1, -2), rtol=1e-5, atol=1e-5)
    assert (k.grad if first else q.grad) is None
    one = native.window_matmul_backward(q0, k0.transpose(-1, -2), w, 2 * att, first, not first)
    assert one[1 if first else 0] is None and one[0 if first else 1] is not None

    a = a0.clone().requires_grad_(first)
    v = v0.clone().requires_grad_(not first)
    unwindow_matmul(a, v, w).square().sum().backward()
    out = native.unwindow_matmul_forward(a0, v0, w)
    ga, gv = native.unwindow_matmul_backward(a0, v0, w, 2 * out)
    torch.testing.assert_close(a.grad if first else v.grad, ga if first else gv, rtol=1e-5, atol=1e-5)
    assert (v.grad if first else a.grad) is None
    one = native.unwindow_matmul_backward(a0, v0, w, 2 * out, need_src=first, need_other=not first)
    assert one[1 if first else 0] is None and one[0 if first else 1] is not None


def test_ops_follow_the_current_stream(device):
    """Launches go to torch's current stream: the same chain on two side streams at once, each ordered
    only by its own stream, gives the result of the default stream (no hidden use of stream 0)."""
    from window_matmul import unwindow_matmul, window_matmul

    B, M, N, w = 4, 1024, 64, 24
    q, k, v = (seeded((B, M, N), s, torch.bfloat16).to(device) for s in (41, 42, 43))

    def chain(x):
        att = window_matmul(x, k.transpose(-1, -2), w)
        return unwindow_matmul(torch.softmax(att.float() * 0.125, -1).to(att.dtype), v, w)

    want = chain(q)
    want2 = chain(q + 1)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(s1):
        got = chain(q)
    with torch.cuda.stream(s2):
        got2 = chain(q + 1)
    s1.synchronize()
    s2.synchronize()
    assert torch.equal(got, want) and torch.equal(got2, want2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_views_at_a_misaligned_storage_offset(device, dtype):
    """Contiguous tensors whose data pointer is not 16-byte aligned (views that start one element
    into a buffer): the ops, the band softmax and the fused attention give the numbers of aligned
    copies, and the fused call does not refuse them."""
    from window_matmul import band_softmax, unwindow_matmul, window_attention, window_matmul

    B, M, N, w = 2, 200, 64, 6

    def shifted(t):
        flat = torch.empty(t.numel() + 1, dtype=t.dtype, device=t.device)
        view = flat[1:].view(t.shape)
        view.copy_(t)
        assert view.is_contiguous() and view.data_ptr() % 16 != 0
        return view

    q, k, v = (seeded((B, M, N), s, dtype).to(device) for s in (61, 62, 63))
    att = window_matmul(q, k.transpose(1, 2), w)
    assert torch.equal(window_matmul(shifted(q), shifted(k).transpose(1, 2), w), att)
    probs = band_softmax(att, 0.125)
    assert torch.equal(band_softmax(shifted(att), 0.125), probs)
    out = unwindow_matmul(probs, v, w)
    assert torch.equal(unwindow_matmul(shifted(probs), shifted(v), w), out)
    if dtype != torch.float32:
        fused = window_attention(q, k, v, w, 0.125)
        assert torch.equal(window_attention(shifted(q), shifted(k), shifted(v), w, 0.125), fused)


@pytest.mark.parametrize("dtype,N", [(torch.bfloat16, 3), (torch.bfloat16, 40), (torch.float16, 72), (torch.float16, 100),
                                      (torch.float32, 3), (torch.float32, 20), (torch.float32, 50), (torch.float32, 121),
                                      (torch.bfloat16, 160), (torch.float16, 256), (torch.bfloat16, 136), (torch.float32, 200)],
                         ids=lambda x: str(x).replace("torch.", ""))
@pytest.mark.parametrize("w", [2, 9, 40, 300])
def test_head_widths_between_the_tuned_ones(device, dtype, N, w):
    """A head width that is not a multiple of 16 (16-bit storage) or 8 (float32) is padded with zero
    columns inside the extension, one beyond 128 is worked on in slices of 128 columns (float32 band
    gradients summed over the slices); results, shapes, contiguity and all four gradients are those of
    the operation on the whole tensors (CPU oracle).  16-bit storage takes the padded and sliced route
    at every window; float32 takes it above w = 256 (w = 300 here, with a longer sequence) and runs the
    tile kernels, which need neither, at the narrower windows."""
    from window_matmul import unwindow_matmul, window_matmul

    B, M = (3, 150) if w < 256 else (2, 700)
    tol = dict(rtol=1e-3, atol=1e-3) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    q, k, v = (seeded((B, M, N), 400 + s, dtype) for s in range(3))
    a = seeded((B, M, 2 * w + 1), 410, dtype, 0.25)
    g_att, g_out = seeded((B, M, 2 * w + 1), 411, dtype, 0.25), seeded((B, M, N), 412, dtype)
    dq, dk, dv, da = (t.clone().to(device).requires_grad_(True) for t in (q, k, v, a))
    att = window_matmul(dq, dk.transpose(1, 2), w)
    out = unwindow_matmul(da, dv, w)
    assert att.shape == (B, M, 2 * w + 1) and out.shape == (B, M, N) and out.is_contiguous()
    att.backward(g_att.to(device))
    out.backward(g_out.to(device))
    f = lambda t: t.float()  # noqa: E731
    ktc = f(k).transpose(1, 2).contiguous()
    torch.testing.assert_close(f(att).cpu(), oracle.window_matmul_forward(f(q), ktc, w), **tol)
    torch.testing.assert_close(f(out).cpu(), oracle.unwindow_matmul_forward(f(a), f(v), w), **tol)
    want_q, want_k = oracle.window_matmul_backward(f(q), ktc, w, f(g_att))
    want_a, want_v = oracle.unwindow_matmul_backward(f(a), f(v), w, f(g_out))
    assert dq.grad.shape == q.shape and dk.grad.shape == k.shape and dv.grad.shape == v.shape
    torch.testing.assert_close(f(dq.grad).cpu(), want_q, **tol)
    torch.testing.assert_close(f(dk.grad).cpu(), want_k.transpose(1, 2), **tol)
    torch.testing.assert_close(f(da.grad).cpu(), want_a, **tol)
    torch.testing.assert_close(f(dv.grad).cpu(), want_v, **tol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32, torch.float64],
                         ids=lambda d: str(d).split(".")[-1])
def test_key_rows_from_contiguous_transposed_keys(device, dtype):
    """Keys given as a contiguous (B,N,M) tensor (reference window_matmul.py:30-40 takes exactly that
    shape) are copied into key rows by the library's own transpose: bit-exact against torch's copy at
    ragged and tile-sized shapes, with a row stride, and the ops on top of it give the same bits as with
    keys that were row-major all along.  Layouts it does not take report WM_ERR_UNSUPPORTED."""
    import wm_ctypes as abi
    from window_matmul import window_matmul

    for B, N, M in ((3, 64, 300), (2, 128, 64), (5, 16, 1), (1, 80, 4097), (2, 8, 129), (7, 48, 1000), (2, 64, 3001)):
        kt = seeded((B, N, M), 201, dtype).to(device)
        assert torch.equal(abi.key_rows(kt), kt.transpose(1, 2).contiguous())
        for off in (8, 3):  # rows that start on a 16-byte boundary, and rows that do not
            view = seeded((B, N, M + 24), 202, dtype).to(device)[:, :, off:off + M]
            assert torch.equal(abi.key_rows(view), view.transpose(1, 2).contiguous())
    # through the Python API: same bits as with row-major keys, forward and both gradients
    B, M, N, w = 3, 333, 64, 21
    q = seeded((B, M, N), 203, dtype).to(device).requires_grad_(True)
    k_rows = seeded((B, M, N), 204, dtype).to(device)
    kt = k_rows.transpose(1, 2).contiguous().requires_grad_(True)      # contiguous (B,N,M)
    kv = k_rows.clone().requires_grad_(True)
    ga = seeded((B, M, 2 * w + 1), 205, dtype).to(device)
    a1 = window_matmul(q, kt, w)
    a1.backward(ga)
    g1 = (q.grad.clone(), kt.grad.clone())
    q.grad = None
    a2 = window_matmul(q, kv.transpose(1, 2), w)
    a2.backward(ga)
    assert torch.equal(a1, a2) and torch.equal(g1[0], q.grad) and torch.equal(g1[1], kv.grad.transpose(1, 2))
    # not taken: a head width whose rows cannot be 16-byte pieces, keys whose unit stride is not along M
    L = abi.lib()
    thin = seeded((2, 3, 64), 207, dtype).to(device)
    out = torch.empty(2, 64, 3, dtype=dtype, device=device)
    assert L.wm_key_rows(abi.op(thin), ctypes.c_void_p(out.data_ptr()), 2, 3, 64, abi.DTYPES[dtype], None) == 7
    rows = seeded((2, 64, 64), 208, dtype).to(device).transpose(1, 2)
    out = torch.empty(2, 64, 64, dtype=dtype, device=device)
    assert L.wm_key_rows(abi.op(rows), ctypes.c_void_p(out.data_ptr()), 2, 64, 64, abi.DTYPES[dtype], None) == 7
