"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py).

CPU part: the oracle reproduces every stored array bit for bit (a regression guard for the
oracle; the stored values were checked against the reference's compiled CPU path when they
were written).  GPU part: the HIP path, through the Python API, against the stored values.
"""
import glob
import os

import numpy as np
import pytest
import torch

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))
DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}
TOL = {"f32": 1e-3, "bf16": 2e-2, "f16": 2e-2}


def load(path):
    z = np.load(path, allow_pickle=False)
    t = {k: torch.from_numpy(z[k]) for k in z.files if z[k].ndim == 3}
    meta = {k: int(z[k]) for k in ("B", "M", "N", "w")}
    return t, meta, str(z["dtype"]), bool(z["checked_against_reference"])


def test_fixtures_exist_and_were_checked_against_the_reference():
    assert len(FIXTURES) == 8
    for path in FIXTURES:
        assert load(path)[3], path


@pytest.mark.parametrize("path", FIXTURES, ids=lambda p: os.path.basename(p)[:-4])
def test_oracle_reproduces_fixture(path):
    t, m, _, _ = load(path)
    w = m["w"]
    kt = t["k"].transpose(1, 2).contiguous()
    assert torch.equal(oracle.window_matmul_forward(t["q"], kt, w), t["att"])
    assert torch.equal(oracle.unwindow_matmul_forward(t["band"], t["v"], w), t["out"])
    ga, gv = oracle.unwindow_matmul_backward(t["band"], t["v"], w, t["grad_o"])
    assert torch.equal(ga, t["grad_band"]) and torch.equal(gv, t["grad_v"])
    gq, gkt = oracle.window_matmul_backward(t["q"], kt, w, t["grad_a_up"])
    assert torch.equal(gq, t["grad_q"]) and torch.equal(gkt, t["grad_kt"])
    # and the independent dense formulation agrees to float32 rounding
    torch.testing.assert_close(oracle.dense_window_matmul(t["q"], kt, w).float(), t["att"], rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(oracle.dense_unwindow_matmul(t["band"], t["v"], w).float(), t["out"], rtol=1e-4, atol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("path", FIXTURES, ids=lambda p: os.path.basename(p)[:-4])
def test_hip_path_matches_fixture(device, path):
    from window_matmul import unwindow_matmul, window_matmul

    t, m, dname, _ = load(path)
    w, tol, dt = m["w"], TOL[dname], DT[dname]
    d = {k: v.to(dt).to(device) for k, v in t.items()}
    q, k, v, band = (d[n].clone().requires_grad_(True) for n in ("q", "k", "v", "band"))
    att = window_matmul(q, k.transpose(1, 2), w)
    att.backward(d["grad_a_up"])
    out = unwindow_matmul(band, v, w)
    out.backward(d["grad_o"])
    mask = oracle.band_mask(m["M"], w, device)
    got = dict(att=att, out=out, grad_band=band.grad, grad_v=v.grad, grad_q=q.grad, grad_kt=k.grad.transpose(1, 2))
    for name, val in got.items():
        torch.testing.assert_close(val.detach().float().cpu(), t[name], rtol=tol, atol=tol, msg=lambda s: f"{name}: {s}")
    for band_out in (att, band.grad):
        outside = band_out.detach()[:, ~mask]
        assert torch.equal(outside, torch.zeros_like(outside)) and not torch.signbit(outside).any()
