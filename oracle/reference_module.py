"""Loader for the reference's own compiled CPU path.  TEST INFRASTRUCTURE ONLY.

``oracle/build_ref.sh`` compiles the reference's dispatcher and scalar CPU
kernels from their sources into ``oracle/_ref/window_matmul_kernel_ref.so``
(a pybind module with the reference's four functions, reference
csrc/window_matmul/window_matmul.cpp:100-106).  Where that file exists this
returns the imported module, otherwise ``None``.
"""
import importlib.util
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_CACHE = []


def reference_module():
    if _CACHE:
        return _CACHE[0]
    path = os.path.join(_HERE, "_ref", "window_matmul_kernel_ref.so")
    mod = None
    if os.path.exists(path):
        import torch  # noqa: F401  (the module links against libtorch)

        spec = importlib.util.spec_from_file_location("window_matmul_kernel_ref", path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
    _CACHE.append(mod)
    return mod
