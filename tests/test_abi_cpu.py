"""Host-side checks that need no GPU: the library loads, exports what the header
declares, validates arguments before touching the device, and the Python layer
mirrors the reference's surface and error behaviour."""
import ctypes
import os
import inspect

import pytest
import torch

import wm_ctypes as abi


def test_library_exports_every_declared_symbol():
    L = abi.lib()
    names = abi.declared_symbols()
    assert {"wm_window_matmul_forward", "wm_window_matmul_backward", "wm_unwindow_matmul_forward",
            "wm_unwindow_matmul_backward", "wm_band_softmax_forward", "wm_band_softmax_backward",
            "wm_band_softmax_kernel_choice", "wm_window_attention_forward", "wm_window_attention_backward",
            "wm_window_attention_supported", "wm_window_attention_backward_static",
            "wm_kernel_choice", "wm_key_rows", "wm_status_string", "wm_abi_version"} <= set(names)
    for name in names:
        assert hasattr(L, name), name
    assert L.wm_abi_version() == 4


def test_argument_validation_happens_on_the_host():
    L = abi.lib()
    dummy = abi.Operand(ctypes.c_void_p(16), 0, 0, 0)
    null = abi.Operand(None, 0, 0, 0)
    P = ctypes.byref
    # empty problems are a no-op, whatever the pointers
    assert L.wm_window_matmul_forward(None, None, None, 0, 4, 4, 1, 0, 0, None) == 0
    assert L.wm_unwindow_matmul_forward(None, None, None, 2, 0, 4, 1, 0, 0, None) == 0
    assert L.wm_window_matmul_backward(None, None, None, None, None, 2, 4, 0, 1, 0, 0, None) == 0
    # status codes from include/window_matmul_hip.h
    assert L.wm_window_matmul_forward(P(dummy), P(dummy), P(null), 1, 4, 4, 1, 0, 0, None) == 1
    assert L.wm_window_matmul_forward(None, P(dummy), P(dummy), 1, 4, 4, 1, 0, 0, None) == 1
    assert L.wm_window_matmul_forward(P(dummy), P(dummy), P(dummy), -1, 4, 4, 1, 0, 0, None) == 2
    assert L.wm_window_matmul_forward(P(dummy), P(dummy), P(dummy), 1, 4, 4, -3, 0, 0, None) == 2
    assert L.wm_window_matmul_forward(P(dummy), P(dummy), P(dummy), 1, 2**31, 4, 1, 0, 0, None) == 2
    assert L.wm_window_matmul_forward(P(dummy), P(dummy), P(dummy), 1, 4, 4, 1, 7, 0, None) == 3
    assert L.wm_unwindow_matmul_backward(P(dummy), P(dummy), P(dummy), P(dummy), P(dummy), 1, 4, 4, 1, 0, 0x80, None) == 4
    assert L.wm_unwindow_matmul_backward(P(dummy), P(dummy), None, P(dummy), P(dummy), 1, 4, 4, 1, 0, 0, None) == 1
    assert b"dtype" in L.wm_status_string(3)
    assert L.wm_status_string(0) == b"ok"


def test_kernel_choice_names():
    L = abi.lib()
    assert L.wm_kernel_choice(1, 2, 128, 64, 4, 0, 1, abi.FORCE_STRIDED) == b"strided_p1"
    assert L.wm_kernel_choice(3, 2, 128, 64, 4, 3, 1, 0) == b"tile_p3"  # float64: tiles on the float64 matrix instruction
    assert L.wm_kernel_choice(1, 2, 128, 7, 0, 3, 0, 0) == b"tile_p1"   # every layout and head width
    assert L.wm_kernel_choice(2, 2, 128, 7, 4, 2, 1, 0) == b"tile_p2"   # bf16 at a head width no tuned kernel takes
    assert L.wm_kernel_choice(1, 2, 128, 64, 4, 0, 0, 0) == b"tile_p1"  # float32 in a layout no tuned kernel takes
    assert L.wm_kernel_choice(2, 2, 128, 64, 4, 3, 1, abi.FORCE_STRIDED) == b"strided_p2"
    assert L.wm_kernel_choice(9, 2, 128, 64, 4, 0, 1, 0) == b"invalid"
    # per family: float32 MFMA, 16-bit wide band, 16-bit narrow band (P1 any w <= 32, P2 and P3 for w % 4 == 0)
    assert L.wm_kernel_choice(1, 7, 3001, 80, 1500, 0, 1, 0) == b"f32_split_p1"  # float32 on the bf16 matrix instruction
    assert L.wm_kernel_choice(1, 7, 3001, 80, 1500, 0, 1, abi.NO_SPLIT_F32) == b"f32_mfma_p1"
    assert L.wm_kernel_choice(3, 7, 3001, 80, 15, 0, 1, 0) == b"f32_mfma_p3"     # below w = 16: the float32 instruction
    assert L.wm_kernel_choice(2, 96, 4096, 32, 64, 0, 1, 0) == b"f32_mfma_p2"    # one 32-column block: no gain from the split
    assert L.wm_kernel_choice(3, 96, 4096, 32, 64, 0, 1, 0) == b"f32_split_p3"
    assert L.wm_kernel_choice(2, 96, 4096, 64, 256, 2, 1, 0) == b"mfma_p2"
    assert L.wm_kernel_choice(1, 96, 16384, 64, 8, 2, 1, 0) == b"narrow_p1"
    assert L.wm_kernel_choice(2, 96, 16384, 64, 8, 1, 1, 0) == b"narrow_p2"
    assert L.wm_kernel_choice(2, 96, 16384, 64, 9, 2, 1, 0) == b"narrow_p2"   # re-pitched LDS image
    assert L.wm_kernel_choice(2, 96, 16384, 64, 13, 2, 1, 0) == b"narrow_p2"
    assert L.wm_kernel_choice(3, 96, 16384, 64, 8, 2, 1, 0) == b"narrow_p3"
    assert L.wm_kernel_choice(3, 96, 16384, 64, 10, 2, 1, 0) == b"narrow_p3"
    # from w = 16 (band-in) / 13 (transposed band-in) at N = 64 the wide-band kernels that load their
    # tiles straight into LDS are faster; without them the narrow kernels keep their old range
    assert L.wm_kernel_choice(2, 96, 16384, 64, 15, 2, 1, 0) == b"narrow_p2"
    assert L.wm_kernel_choice(2, 96, 16384, 64, 16, 2, 1, 0) == b"mfma_p2"
    assert L.wm_kernel_choice(3, 96, 16384, 64, 13, 2, 1, 0) == b"mfma_p3"
    assert L.wm_kernel_choice(3, 96, 16384, 64, 27, 2, 1, 0) == b"mfma_p3"
    assert L.wm_kernel_choice(3, 96, 16384, 64, 27, 2, 1, abi.NO_LDS_DIRECT) == b"narrow_p3"
    assert L.wm_kernel_choice(3, 96, 16384, 64, 30, 2, 1, abi.NO_LDS_DIRECT) == b"mfma_p3"  # two workgroups per CU: slower
    assert L.wm_kernel_choice(2, 96, 16384, 64, 32, 2, 1, abi.NO_LDS_DIRECT) == b"narrow_p2"  # 32 rows per wave still fit LDS
    assert L.wm_kernel_choice(2, 96, 16384, 32, 32, 2, 1, 0) == b"narrow_p2"
    assert L.wm_kernel_choice(3, 96, 16384, 32, 28, 2, 1, 0) == b"mfma_p3"
    assert L.wm_kernel_choice(2, 96, 16384, 128, 12, 1, 1, 0) == b"mfma_p2"
    assert L.wm_kernel_choice(3, 96, 16384, 128, 32, 2, 1, 0) == b"mfma_p3"   # images beyond 64 KB of LDS
    assert L.wm_kernel_choice(1, 96, 16384, 64, 8, 2, 1, abi.NO_NARROW_BAND) == b"mfma_p1"
    # the band-out kernel of the narrow family reaches w = 63 while the operands fit the registers (N <= 64)
    assert L.wm_kernel_choice(1, 96, 16384, 64, 48, 2, 1, 0) == b"narrow_p1"
    assert L.wm_kernel_choice(1, 96, 16384, 48, 63, 1, 1, 0) == b"narrow_p1"
    assert L.wm_kernel_choice(1, 96, 16384, 64, 64, 2, 1, 0) == b"mfma_p1"
    assert L.wm_kernel_choice(1, 96, 16384, 128, 48, 2, 1, 0) == b"mfma_p1"
    assert L.wm_kernel_choice(2, 96, 16384, 64, 48, 2, 1, 0) == b"mfma_p2"
    # the narrowest windows (w <= 3, not enough terms for a matrix pipe): vector-ALU band-in kernels
    assert L.wm_kernel_choice(2, 96, 16384, 64, 1, 2, 1, 0) == b"vector_p2"
    assert L.wm_kernel_choice(3, 96, 16384, 64, 3, 1, 1, 0) == b"vector_p3"
    assert L.wm_kernel_choice(1, 96, 16384, 64, 7, 1, 1, 0) == b"narrow_p1"
    assert L.wm_kernel_choice(1, 96, 16384, 64, 2, 2, 1, 0) == b"narrow_p1"
    assert L.wm_kernel_choice(1, 96, 16384, 64, 3, 2, 1, 0) == b"narrow_p1"
    assert L.wm_kernel_choice(2, 96, 16384, 64, 7, 2, 1, abi.NO_NARROW_BAND) == b"tile_p2"   # below the wide-band kernels' w = 8
    # float32: band-in products on the vector ALU up to w = 14, the float32 MFMA kernels beyond; the
    # band-out product on the narrow-band MFMA kernel up to w = 31 when N is a multiple of 16 up to 64
    assert L.wm_kernel_choice(2, 96, 16384, 64, 3, 0, 1, 0) == b"vector_p2"
    assert L.wm_kernel_choice(1, 2, 128, 64, 4, 0, 1, 0) == b"narrow_p1"
    assert L.wm_kernel_choice(1, 2, 128, 48, 31, 0, 1, 0) == b"narrow_p1"
    assert L.wm_kernel_choice(1, 2, 128, 64, 32, 0, 1, 0) == b"f32_split_p1"
    assert L.wm_kernel_choice(1, 2, 128, 128, 4, 0, 1, 0) == b"vector_p1"
    assert L.wm_kernel_choice(1, 2, 128, 24, 4, 0, 1, 0) == b"vector_p1"
    assert L.wm_kernel_choice(3, 96, 16384, 64, 11, 0, 1, 0) == b"vector_p3"
    assert L.wm_kernel_choice(3, 96, 16384, 32, 14, 0, 1, 0) == b"vector_p3"
    assert L.wm_kernel_choice(3, 96, 16384, 128, 15, 0, 1, 0) == b"f32_mfma_p3"
    # float32 band-in products on the narrow-band MFMA kernels: N a multiple of 16 up to 64, w = 12 (15) .. 28
    assert L.wm_kernel_choice(3, 96, 16384, 64, 12, 0, 1, 0) == b"narrow_p3"
    assert L.wm_kernel_choice(2, 96, 16384, 32, 15, 0, 1, 0) == b"narrow_p2"
    assert L.wm_kernel_choice(2, 96, 16384, 16, 28, 0, 1, 0) == b"narrow_p2"
    assert L.wm_kernel_choice(2, 96, 16384, 64, 29, 0, 1, 0) == b"f32_split_p2"
    assert L.wm_kernel_choice(2, 96, 16384, 64, 29, 0, 1, abi.NO_SPLIT_F32) == b"f32_mfma_p2"
    assert L.wm_kernel_choice(1, 96, 16384, 64, 8, 0, 1, abi.NO_NARROW_BAND) == b"f32_mfma_p1"
    assert L.wm_kernel_choice(1, 2, 128, 3, 4, 0, 1, 0) == b"tile_p1"  # N not a multiple of 8
    assert L.wm_kernel_choice(1, 2, 128, 64, 4, 2, 0, 0) == b"tile_p1"  # layout not vector friendly


def test_python_surface_matches_reference():
    import window_matmul
    from window_matmul.window_matmul import UnwindowMatmulFunc, WindowMatmulFunc

    assert window_matmul.__all__ == ["window_matmul", "unwindow_matmul"]
    for fn in (window_matmul.window_matmul, window_matmul.unwindow_matmul):
        assert list(inspect.signature(fn).parameters) == ["inp", "other", "window_size"]
    for cls in (WindowMatmulFunc, UnwindowMatmulFunc):
        assert issubclass(cls, torch.autograd.Function)

    import window_matmul_kernel as native

    for name in ("window_matmul_forward", "window_matmul_backward", "unwindow_matmul_forward",
                 "unwindow_matmul_backward"):
        assert callable(getattr(native, name))


def test_window_size_zero_paths_are_plain_torch():
    """w = 0 never reaches the kernels (reference window_matmul.py:33-34, 69-70; tests/test_attention.py:75-87)."""
    from window_matmul import unwindow_matmul, window_matmul

    q = torch.randn(2, 3, 5, 4)
    k = torch.randn(2, 3, 5, 4)
    v = torch.randn(2, 3, 5, 4)
    att = window_matmul(q, k.transpose(-1, -2), 0)
    assert att.shape == (2, 3, 5, 1)
    torch.testing.assert_close(att[..., 0], (q * k).sum(-1))
    out = unwindow_matmul(att.softmax(-1), v, None)
    torch.testing.assert_close(out, v)


def test_native_module_rejects_cpu_tensors_and_bad_shapes():
    """Errors surface as RuntimeError with the reference's texts (reference cuda/utils.cuh:3-4)."""
    import window_matmul_kernel as native

    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        native.window_matmul_forward(torch.zeros(1, 4, 3), torch.zeros(1, 3, 4), 1)
    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        native.unwindow_matmul_backward(torch.zeros(1, 4, 3), torch.zeros(1, 4, 3), 1, torch.zeros(1, 4, 3))


def test_only_one_hip_runtime_is_mapped():
    import window_matmul_kernel  # noqa: F401

    paths = {line.split()[-1] for line in open("/proc/self/maps") if "libamdhip64" in line}
    assert len(paths) == 1, paths


def test_setup_py_builds_an_importable_tree(tmp_path):
    """setup.py (packaging in the manner of reference setup.py:22-116) produces a directory from
    which the package and its native module import without any sys.path help from this repo."""
    import subprocess
    import sys

    pkg = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "pytorch-window-matmul_amd")
    subprocess.check_call([sys.executable, "setup.py", "-q", "build", "--build-base", str(tmp_path)], cwd=pkg)
    (lib,) = [d for d in os.listdir(tmp_path) if d.startswith("lib")]
    code = ("import window_matmul, window_matmul_kernel, wm_ctypes; "
            "assert window_matmul.__all__ == ['window_matmul', 'unwindow_matmul']; "
            "assert window_matmul_kernel.abi_version() == wm_ctypes.lib().wm_abi_version(); "
            "print(window_matmul.__file__)")
    out = subprocess.check_output([sys.executable, "-c", code], cwd=str(tmp_path),
                                  env={**os.environ, "PYTHONPATH": os.path.join(str(tmp_path), lib)}, text=True)
    assert str(tmp_path) in out
