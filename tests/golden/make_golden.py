#!/usr/bin/env python3
"""Writes the golden fixtures next to this file (run from the repository root).

Each fixture is one ``.npz`` with the inputs and the expected outputs of the four ops
for one workload: BASELINE config 1 at its exact shape and shrunken versions of configs
2-5 (same dtypes, same edge structure, sizes the CPU loops finish in a second).

Expected values come from the C restatement in ``oracle/`` run in float32 on the inputs
after rounding them to the workload's storage dtype.  Where the reference's own compiled
CPU path is available (``oracle/_ref``, built from the reference sources in this
container) every expected array is checked to be bit-identical to it before it is
written, and the fixture records that in ``checked_against_reference``.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, REPO)

import oracle  # noqa: E402

ROUND = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}

# name: (B, M, N, w, storage dtype, what is special)
CASES = {
    "c1_plumbing_f32": dict(B=2, M=128, N=64, w=4, dtype="f32"),
    "c2_small_window_bf16": dict(B=1, M=300, N=64, w=8, dtype="bf16"),
    "c3_local_attention_bf16": dict(B=1, M=200, N=64, w=96, dtype="bf16", qk_scale=0.125),
    "c4_wide_head_f16": dict(B=1, M=200, N=128, w=48, dtype="f16", uniform_band=True),
    "c5_ragged_w1_f32": dict(B=1, M=151, N=80, w=1, dtype="f32", zero_rows=True),
    "c5_ragged_w33_f32": dict(B=1, M=151, N=80, w=33, dtype="f32", zero_rows=True),
    "c5_ragged_w75_bf16": dict(B=1, M=151, N=80, w=75, dtype="bf16", zero_rows=True),
    # float32 with a band that covers most of the sequence, over more than two 128-row tiles
    "c5_ragged_w150_f32": dict(B=1, M=301, N=80, w=150, dtype="f32", zero_rows=True),
}


def build(name, cfg, seed):
    B, M, N, w = cfg["B"], cfg["M"], cfg["N"], cfg["w"]
    g = torch.Generator().manual_seed(seed)
    rnd = ROUND[cfg["dtype"]]

    def draw(*shape, scale=1.0):
        return (torch.randn(*shape, generator=g) * scale).to(rnd).float()

    s = cfg.get("qk_scale", 1.0)
    q, k, v, grad_o = draw(B, M, N, scale=s), draw(B, M, N, scale=s), draw(B, M, N), draw(B, M, N)
    if cfg.get("zero_rows"):
        rows = torch.randperm(M, generator=g)[: max(1, M // 20)]
        q[:, rows] = 0.0
    kt = k.transpose(1, 2).contiguous()
    att = oracle.window_matmul_forward(q, kt, w)
    if cfg.get("uniform_band"):
        band = torch.rand(B, M, 2 * w + 1, generator=g)
        band = (band / band.sum(-1, keepdim=True)).to(rnd).float()
    else:
        band = att.softmax(-1).to(rnd).float()
    grad_a_up = draw(B, M, 2 * w + 1, scale=0.25)
    out = oracle.unwindow_matmul_forward(band, v, w)
    grad_band, grad_v = oracle.unwindow_matmul_backward(band, v, w, grad_o)
    grad_q, grad_kt = oracle.window_matmul_backward(q, kt, w, grad_a_up)
    expected = dict(att=att, out=out, grad_band=grad_band, grad_v=grad_v, grad_q=grad_q, grad_kt=grad_kt)
    ref = oracle.reference_module()
    checked = False
    if ref is not None:
        theirs = dict(att=ref.window_matmul_forward(q, kt, w), out=ref.unwindow_matmul_forward(band, v, w))
        theirs["grad_band"], theirs["grad_v"] = ref.unwindow_matmul_backward(band, v, w, grad_o)
        theirs["grad_q"], theirs["grad_kt"] = ref.window_matmul_backward(q, kt, w, grad_a_up)
        for key, val in expected.items():
            assert torch.equal(val, theirs[key]), (name, key)
        checked = True
    arrays = dict(q=q, k=k, v=v, band=band, grad_o=grad_o, grad_a_up=grad_a_up, **expected)
    meta = dict(B=B, M=M, N=N, w=w)
    np.savez_compressed(
        os.path.join(HERE, name + ".npz"),
        dtype=np.array(cfg["dtype"]), checked_against_reference=np.array(checked),
        **{k_: np.array(v_) for k_, v_ in meta.items()},
        **{k_: v_.numpy() for k_, v_ in arrays.items()},
    )
    return checked


if __name__ == "__main__":
    only = sys.argv[1:]  # fixture names to (re)write; all of them when none is given
    for n, (name, cfg) in enumerate(CASES.items()):
        if only and name not in only:
            continue
        ok = build(name, cfg, seed=1000 + n)
        print(f"{name}: written (bit-identical to the compiled reference: {ok})")
