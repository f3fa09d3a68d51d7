"""ctypes binding of libwindow_matmul_hip.so (mirrors include/window_matmul_hip.h).

For callers that want the C ABI without the PyTorch extension in between: the tests,
the benchmark's per-kernel timing, and as a template for bindings from other hosts.
Tensors are only used as (pointer, strides) carriers; work is enqueued on torch's
current stream."""
import ctypes
import os
import re

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(HERE)
LIB_PATH = os.environ.get("WM_LIBRARY_PATH", os.path.join(HERE, "libwindow_matmul_hip.so"))
HEADER = os.path.join(REPO, "include", "window_matmul_hip.h")

DTYPES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2, torch.float64: 3}
FORCE_STRIDED = 0x1
NO_ALIGNED_BAND = 0x2
NO_NARROW_BAND = 0x4
NO_LDS_DIRECT = 0x8
NO_SPLIT_F32 = 0x10


class Operand(ctypes.Structure):
    _fields_ = [
        ("data", ctypes.c_void_p),
        ("stride_b", ctypes.c_int64),
        ("stride_r", ctypes.c_int64),
        ("stride_c", ctypes.c_int64),
    ]


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(wm_[a-z_0-9]+)\s*\(", text)))


_LIB = None


def lib():
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(f"{LIB_PATH} is not built; run python pytorch-window-matmul_amd/build.py")
        L = ctypes.CDLL(LIB_PATH)
        P, i64, u32, vp = ctypes.POINTER(Operand), ctypes.c_int64, ctypes.c_uint, ctypes.c_void_p
        tail = [i64, i64, i64, i64, ctypes.c_int, u32, vp]
        L.wm_window_matmul_forward.argtypes = [P, P, P] + tail
        L.wm_unwindow_matmul_forward.argtypes = [P, P, P] + tail
        L.wm_window_matmul_backward.argtypes = [P, P, P, P, P] + tail
        L.wm_unwindow_matmul_backward.argtypes = [P, P, P, P, P] + tail
        L.wm_status_string.restype = ctypes.c_char_p
        L.wm_status_string.argtypes = [ctypes.c_int]
        L.wm_kernel_choice.restype = ctypes.c_char_p
        L.wm_kernel_choice.argtypes = [ctypes.c_int, i64, i64, i64, i64, ctypes.c_int, ctypes.c_int, u32]
        sm_tail = [i64, i64, i64, ctypes.c_double, ctypes.c_int, ctypes.c_int, u32, vp]
        L.wm_band_softmax_forward.argtypes = [P, P] + sm_tail
        L.wm_band_softmax_backward.argtypes = [P, P, P] + sm_tail
        L.wm_band_softmax_kernel_choice.restype = ctypes.c_char_p
        L.wm_band_softmax_kernel_choice.argtypes = [i64, ctypes.c_int, ctypes.c_int, ctypes.c_int, u32]
        L.wm_window_attention_forward.argtypes = [P, P, P, P, vp, i64, i64, i64, i64, ctypes.c_double, ctypes.c_int,
                                                  ctypes.c_int, u32, vp]
        L.wm_window_attention_backward.argtypes = [P, P, P, P, vp, P, P, P, P, vp, i64, i64, i64, i64, ctypes.c_double,
                                                   ctypes.c_int, u32, vp]
        L.wm_window_attention_backward_static.argtypes = [P, P, P, P, vp, P, P, P, P, i64, i64, i64, i64,
                                                          ctypes.c_double, ctypes.c_int, u32, vp]
        L.wm_window_attention_supported.argtypes = [i64, i64, i64, ctypes.c_int, ctypes.c_double]
        L.wm_key_rows.argtypes = [P, vp, i64, i64, i64, ctypes.c_int, vp]
        _LIB = L
    return _LIB


def op(t):
    """Operand for a rank-3 tensor (None -> NULL pointer)."""
    if t is None:
        return None
    assert t.dim() == 3
    return ctypes.byref(Operand(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2)))


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(status, what):
    if status != 0:
        raise RuntimeError(f"{what}: {lib().wm_status_string(status).decode()} ({status})")


def window_forward(q, k, w, flags=0, out=None):
    """q (B,M,N), k (B,N,M) (any strides) -> a (B,M,2w+1)."""
    B, M, N = q.shape
    a = torch.empty(B, M, 2 * w + 1, dtype=q.dtype, device=q.device) if out is None else out
    _check(lib().wm_window_matmul_forward(op(q), op(k), op(a), B, M, N, w, DTYPES[q.dtype], flags, _stream()),
           "wm_window_matmul_forward")
    return a


def key_rows(k):
    """wm_key_rows: k (B,N,M) with unit stride along M -> contiguous key rows (B,M,N)."""
    B, N, M = k.shape
    rows = torch.empty(B, M, N, dtype=k.dtype, device=k.device)
    _check(lib().wm_key_rows(op(k), ctypes.c_void_p(rows.data_ptr()), B, N, M, DTYPES[k.dtype], _stream()), "wm_key_rows")
    return rows


def window_backward(q, k, w, ga, flags=0, want_q=True, want_k=True):
    B, M, N = q.shape
    gq = torch.empty(B, M, N, dtype=q.dtype, device=q.device) if want_q else None
    gk = torch.empty(B, M, N, dtype=q.dtype, device=q.device).transpose(1, 2) if want_k else None
    _check(lib().wm_window_matmul_backward(op(q), op(k), op(ga), op(gq), op(gk), B, M, N, w, DTYPES[q.dtype], flags,
                                          _stream()), "wm_window_matmul_backward")
    return gq, gk


def unwindow_forward(a, v, w, flags=0):
    B, M, N = v.shape
    o = torch.empty(B, M, N, dtype=v.dtype, device=v.device)
    _check(lib().wm_unwindow_matmul_forward(op(a), op(v), op(o), B, M, N, w, DTYPES[v.dtype], flags, _stream()),
           "wm_unwindow_matmul_forward")
    return o


def unwindow_backward(a, v, w, go, flags=0, want_a=True, want_v=True):
    B, M, N = v.shape
    ga = torch.empty(B, M, 2 * w + 1, dtype=v.dtype, device=v.device) if want_a else None
    gv = torch.empty(B, M, N, dtype=v.dtype, device=v.device) if want_v else None
    _check(lib().wm_unwindow_matmul_backward(op(a), op(v), op(go), op(ga), op(gv), B, M, N, w, DTYPES[v.dtype], flags,
                                            _stream()), "wm_unwindow_matmul_backward")
    return ga, gv


def band_softmax_forward(a, scale=1.0, mask=False, flags=0, out=None):
    """a (B,M,2w+1) -> softmax(scale * a) along the band; out may be a itself."""
    B, M, W = a.shape
    p = torch.empty_like(a) if out is None else out
    _check(lib().wm_band_softmax_forward(op(a), op(p), B, M, W // 2, float(scale), int(mask), DTYPES[a.dtype], flags,
                                        _stream()), "wm_band_softmax_forward")
    return p


def band_softmax_backward(p, gp, scale=1.0, mask=False, flags=0, out=None):
    B, M, W = p.shape
    ga = torch.empty_like(p) if out is None else out
    _check(lib().wm_band_softmax_backward(op(p), op(gp), op(ga), B, M, W // 2, float(scale), int(mask),
                                         DTYPES[p.dtype], flags, _stream()), "wm_band_softmax_backward")
    return ga


UNSUPPORTED = 7


def attention_forward(q, k, v, w, scale=1.0, mask=False, flags=0, want_lse=True):
    """q, k, v (B,M,N) row-major (k holds key rows) -> (o (B,M,N), lse (B,M) float32 or None)."""
    B, M, N = q.shape
    o = torch.empty(B, M, N, dtype=q.dtype, device=q.device)
    lse = torch.empty(B, M, dtype=torch.float32, device=q.device) if want_lse else None
    _check(lib().wm_window_attention_forward(op(q), op(k), op(v), op(o),
                                            ctypes.c_void_p(lse.data_ptr()) if want_lse else None, B, M, N, w,
                                            float(scale), int(mask), DTYPES[q.dtype], flags, _stream()),
           "wm_window_attention_forward")
    return o, lse


STATIC_SCRATCH_ROWS = 1 << 21
SCRATCH_TOO_SMALL = 8


def attention_backward_static(q, k, v, o, lse, go, gq, gk, gv, w, scale=1.0, flags=0):
    """wm_window_attention_backward_static: outputs are the caller's (None skips one), the workspace the
    library's static array; the call itself allocates nothing.  Returns the status code."""
    B, M, N = q.shape
    return lib().wm_window_attention_backward_static(op(q), op(k), op(v), op(o), ctypes.c_void_p(lse.data_ptr()),
                                                     op(go), op(gq), op(gk), op(gv), B, M, N, w, float(scale),
                                                     DTYPES[q.dtype], flags, _stream())


def attention_backward(q, k, v, o, lse, go, w, scale=1.0, flags=0, want=(True, True, True)):
    """Gradients (gq, gk, gv), all (B,M,N) row-major, from the forward's o and lse; None where not wanted."""
    B, M, N = q.shape
    gq, gk, gv = (torch.empty(B, M, N, dtype=q.dtype, device=q.device) if x else None for x in want)
    delta = torch.empty(2, B, M, dtype=torch.float32, device=q.device)
    _check(lib().wm_window_attention_backward(op(q), op(k), op(v), op(o), ctypes.c_void_p(lse.data_ptr()), op(go),
                                             op(gq), op(gk), op(gv), ctypes.c_void_p(delta.data_ptr()), B, M, N, w,
                                             float(scale), DTYPES[q.dtype], flags, _stream()),
           "wm_window_attention_backward")
    return gq, gk, gv
