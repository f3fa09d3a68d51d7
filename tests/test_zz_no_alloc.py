"""wm_window_attention_backward_static, the entry point for callers that cannot allocate device
memory: same kernels as wm_window_attention_backward with the delta workspace in the library's
static device array.  Called through the C ABI twice in a row, the second time on a smaller
problem (the array then still holds the first call's rows), and compared bit for bit with the
existing entry point; float16 / bfloat16 results of the two must not differ at all, which is
tighter than the 2e-2 the fused path is held to against the oracle."""
import math

import pytest
import torch

import wm_ctypes as abi
from conftest import seeded

pytestmark = pytest.mark.gpu

# (B, M, N, w): the second problem is smaller than the first in batch, length and window
# Shapes whose backward is the two-kernel form, which hands D and the log-sum-exp from the first kernel to
# the second through the workspace (wide window; wide head), then one that takes the one-kernel backward,
# which leaves the workspace alone.
CALLS = [(5, 700, 64, 100), (2, 260, 128, 12), (2, 200, 64, 12)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bfloat16", "float16"])
def test_static_workspace_matches_caller_workspace(device, dtype):
    for n, (B, M, N, w) in enumerate(CALLS):
        scale = 1.0 / math.sqrt(N)
        q, k, v, go = (seeded((B, M, N), 900 + 10 * n + s, dtype).to(device) for s in range(4))
        o, lse = abi.attention_forward(q, k, v, w, scale)
        want = abi.attention_backward(q, k, v, o, lse, go, w, scale)
        got = [torch.full_like(q, float("nan")) for _ in range(3)]
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        status = abi.attention_backward_static(q, k, v, o, lse, go, *got, w, scale)
        torch.cuda.synchronize()
        assert status == 0, abi.lib().wm_status_string(status)
        if n > 0:  # the first call on a GPU may still page the library's code and data in
            assert torch.cuda.mem_get_info()[0] == free_before
        for name, g, wnt in zip(("grad_q", "grad_k", "grad_v"), got, want):
            assert torch.equal(g.view(torch.int16), wnt.view(torch.int16)), (name, B, M, N, w)


def test_skipped_gradients_and_the_size_limit(device):
    B, M, N, w = 2, 300, 128, 70
    q, k, v, go = (seeded((B, M, N), 950 + s, torch.float16).to(device) for s in range(4))
    o, lse = abi.attention_forward(q, k, v, w, 0.1)
    _, want_k, _ = abi.attention_backward(q, k, v, o, lse, go, w, 0.1, want=(False, True, False))
    gk = torch.empty_like(k)
    assert abi.attention_backward_static(q, k, v, o, lse, go, None, gk, None, w, 0.1) == 0
    assert torch.equal(gk.view(torch.int16), want_k.view(torch.int16))
    # beyond the static array: refused on the host, nothing launched (the extents are only claimed)
    rows = abi.STATIC_SCRATCH_ROWS
    L = abi.lib()
    status = L.wm_window_attention_backward_static(abi.op(q), abi.op(k), abi.op(v), abi.op(o), lse.data_ptr(),
                                                   abi.op(go), None, abi.op(gk), None, rows // 256 + 1, 256, N, w, 0.1,
                                                   abi.DTYPES[q.dtype], 0, None)
    assert status == abi.SCRATCH_TOO_SMALL
    assert b"WM_STATIC_SCRATCH_ROWS" in L.wm_status_string(status)
    torch.cuda.synchronize()
