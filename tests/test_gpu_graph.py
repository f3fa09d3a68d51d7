"""The ops under HIP graph capture: every kernel is launched on the capturing stream, nothing
synchronises and nothing is cleared with a memset, so a captured chain must replay to the same
bits as the eager run, on every replay and for new contents of the static input buffers."""
import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu


def chain(native, q, kt, v, go, w, scale):
    """Forward and backward of window -> band softmax -> unwindow through the native module."""
    att = native.window_matmul_forward(q, kt, w)
    probs = native.band_softmax_forward(att, scale, False)
    out = native.unwindow_matmul_forward(probs, v, w)
    gp, gv = native.unwindow_matmul_backward(probs, v, w, go)
    ga = native.band_softmax_backward(probs, gp, scale, False)
    gq, gkt = native.window_matmul_backward(q, kt, w, ga)
    return out, gq, gkt, gv


def fused(native, q, k, v, go, w, scale):
    out, lse = native.window_attention_forward(q, k, v, w, scale, False)
    return (out,) + tuple(native.window_attention_backward(q, k, v, out, lse, go, w, scale))


@pytest.mark.parametrize("which", ["separate_ops", "fused_attention"])
@pytest.mark.parametrize("shape", [(3, 300, 64, 40), (2, 500, 64, 8), (2, 400, 64, 64), (2, 400, 64, 100)],
                         ids=["w40", "w8", "w64_dynamic_lds", "w100_two_kernels"])
def test_replay_matches_eager(device, which, shape):
    import window_matmul_kernel as native

    B, M, N, w = shape
    scale = 0.125
    static = [seeded((B, M, N), s, torch.bfloat16).to(device) for s in (91, 92, 93, 94)]
    q, k, v, go = static

    def run():
        if which == "fused_attention":
            return fused(native, q, k, v, go, w, scale)
        return chain(native, q, k.transpose(1, 2), v, go, w, scale)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):  # warm-up outside capture
            run()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run()
    for round_ in range(3):
        for i, t in enumerate(static):  # new contents, same buffers
            t.copy_(seeded((B, M, N), 100 + 10 * round_ + i, torch.bfloat16).to(device))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = run()  # eager work between replays
        torch.cuda.synchronize()
        for x, y in zip(got, want):
            assert torch.equal(x, y)
