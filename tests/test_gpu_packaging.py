"""The installable layout on a GPU: `setup.py build` (packaging in the manner of reference
setup.py:22-116) yields a tree from which `window_matmul` imports with no help from this
repository's paths and runs its kernels.  The shared objects are the prebuilt ones (WM_PREBUILT=1:
nothing is compiled inside the test)."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

CHILD = r"""
import sys, torch, window_matmul, window_matmul_kernel
assert not any(p.rstrip('/').endswith('pytorch-window-matmul_amd') for p in sys.path), sys.path
dev = torch.device('cuda:0')
g = torch.Generator().manual_seed(7)
B, M, N, w = 2, 96, 32, 5
q, k, v = (torch.randn(B, M, N, generator=g).to(dev) for _ in range(3))
att = window_matmul.window_matmul(q, k.transpose(1, 2), w)
dense = torch.bmm(q, k.transpose(1, 2))
i = torch.arange(M, device=dev)[:, None]; j = torch.arange(2 * w + 1, device=dev)[None, :]
c = i + j - w
want = torch.where((c >= 0) & (c < M), dense.gather(2, c.clamp(0, M - 1).expand(B, -1, -1)), torch.zeros((), device=dev))
torch.testing.assert_close(att, want, rtol=1e-3, atol=1e-3)
out = window_matmul.unwindow_matmul(att.softmax(-1), v, w)
assert out.shape == (B, M, N) and torch.isfinite(out).all()
print('ok', window_matmul.__file__, window_matmul_kernel.__file__)
"""


def test_built_tree_runs_on_the_gpu(device, tmp_path):
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    pkg = os.path.join(repo, "pytorch-window-matmul_amd")
    env = {k: v for k, v in os.environ.items() if k != "PYTHONPATH"}
    subprocess.check_call([sys.executable, "setup.py", "-q", "build", "--build-base", str(tmp_path)], cwd=pkg,
                          env={**env, "WM_PREBUILT": "1"})
    (lib,) = [d for d in os.listdir(tmp_path) if d.startswith("lib")]
    out = subprocess.check_output([sys.executable, "-c", CHILD], cwd=str(tmp_path), text=True, timeout=100,
                                  env={**env, "PYTHONPATH": os.path.join(str(tmp_path), lib)})
    assert out.startswith("ok") and out.count(str(tmp_path)) == 2, out
