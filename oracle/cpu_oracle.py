"""ctypes front end of the C restatement (``window_matmul_oracle.c``).

TEST INFRASTRUCTURE ONLY -- the checker, never the thing measured or shipped.

The four functions mirror the reference's native module surface
(reference csrc/window_matmul/window_matmul.cpp:100-106): 3-D CPU tensors in,
freshly allocated tensors out, ``other`` of the window op in the reference's
``(B, N, M)`` orientation.  float32 and float64 run natively; float16/bfloat16
inputs are upcast to float32 first (the reference has no bfloat16 dispatch and
accumulates float16 in half precision, reference cpu:28,43; the comparison
target for reduced precision is the float32 result on the rounded inputs).
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def load_oracle_library(build_if_missing: bool = True) -> ctypes.CDLL:
    """Loads ``libwm_oracle.so``; compiles it with gcc first if it is absent."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = os.path.join(_HERE, "libwm_oracle.so")
    if not os.path.exists(path):
        if not build_if_missing:
            raise FileNotFoundError(path)
        subprocess.check_call(["make", "-C", _HERE, "libwm_oracle.so"])
    lib = ctypes.CDLL(path)
    i64, ptr = ctypes.c_int64, ctypes.c_void_p
    for sfx in ("f32", "f64"):
        getattr(lib, f"wm_oracle_window_fw_{sfx}").argtypes = [ptr, ptr, ptr, i64, i64, i64, i64]
        getattr(lib, f"wm_oracle_unwindow_fw_{sfx}").argtypes = [ptr, ptr, ptr, i64, i64, i64, i64]
        getattr(lib, f"wm_oracle_window_bw_{sfx}").argtypes = [ptr] * 5 + [i64] * 4
        getattr(lib, f"wm_oracle_unwindow_bw_{sfx}").argtypes = [ptr] * 5 + [i64] * 4
        for op in ("window_fw", "unwindow_fw", "window_bw", "unwindow_bw"):
            getattr(lib, f"wm_oracle_{op}_{sfx}").restype = None
    _LIB = lib
    return lib


def _prep(*tensors):
    out = []
    dtype = tensors[0].dtype
    work = torch.float64 if dtype == torch.float64 else torch.float32
    for t in tensors:
        if t.device.type != "cpu":
            raise RuntimeError("oracle runs on CPU tensors only")
        if t.dim() != 3:
            raise RuntimeError("oracle expects 3-D tensors")
        out.append(t.detach().to(work).contiguous())
    return out, ("f64" if work == torch.float64 else "f32"), work


def _check_window(src, other):
    if src.dim() != other.dim() or src.size(-1) != other.size(-2) or src.size(-2) != other.size(-1):
        raise RuntimeError("Input mismatch")  # reference cpu:11-14


def _check_unwindow(src, other, ws):
    if src.dim() != other.dim() or src.size(-1) != 2 * ws + 1 or src.size(-2) != other.size(-2):
        raise RuntimeError("Input mismatch")  # reference cpu:106-109


def window_matmul_forward(src, other, window_size):
    """A = band(Q . K^T);  src (B,M,N), other (B,N,M) -> (B,M,2w+1).  reference cpu:6-50."""
    _check_window(src, other)
    (q, kt), sfx, work = _prep(src, other)
    B, M, N = q.shape
    out = torch.empty(B, M, 2 * window_size + 1, dtype=work)
    fn = getattr(load_oracle_library(), f"wm_oracle_window_fw_{sfx}")
    fn(q.data_ptr(), kt.data_ptr(), out.data_ptr(), B, M, N, window_size)
    return out


def window_matmul_backward(src, other, window_size, grad_output):
    """(dQ (B,M,N), dK^T (B,N,M)).  reference cpu:52-99."""
    _check_window(src, other)
    (q, kt, g), sfx, work = _prep(src, other, grad_output)
    B, M, N = q.shape
    gq = torch.empty(B, M, N, dtype=work)
    gk = torch.empty(B, N, M, dtype=work)
    fn = getattr(load_oracle_library(), f"wm_oracle_window_bw_{sfx}")
    fn(q.data_ptr(), kt.data_ptr(), g.data_ptr(), gq.data_ptr(), gk.data_ptr(), B, M, N, window_size)
    return gq, gk


def unwindow_matmul_forward(src, other, window_size):
    """O = band . V;  src (B,M,2w+1), other (B,M,N) -> (B,M,N).  reference cpu:101-144."""
    _check_unwindow(src, other, window_size)
    (a, v), sfx, work = _prep(src, other)
    B, M, N = v.shape
    out = torch.empty(B, M, N, dtype=work)
    fn = getattr(load_oracle_library(), f"wm_oracle_unwindow_fw_{sfx}")
    fn(a.data_ptr(), v.data_ptr(), out.data_ptr(), B, M, N, window_size)
    return out


def unwindow_matmul_backward(src, other, window_size, grad_output):
    """(dA (B,M,2w+1), dV (B,M,N)).  reference cpu:146-193."""
    _check_unwindow(src, other, window_size)
    (a, v, g), sfx, work = _prep(src, other, grad_output)
    B, M, N = v.shape
    ga = torch.empty(B, M, 2 * window_size + 1, dtype=work)
    gv = torch.empty(B, M, N, dtype=work)
    fn = getattr(load_oracle_library(), f"wm_oracle_unwindow_bw_{sfx}")
    fn(a.data_ptr(), v.data_ptr(), g.data_ptr(), ga.data_ptr(), gv.data_ptr(), B, M, N, window_size)
    return ga, gv
