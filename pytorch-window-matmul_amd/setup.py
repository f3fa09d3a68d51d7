"""Installable packaging of the MI355X build, in the manner of the reference's setup.py
(reference setup.py:22-116: one native module ``window_matmul_kernel`` plus the
``window_matmul`` package), without its CUDA/CPU switch: the only target is gfx950.

    pip install --no-build-isolation ./pytorch-window-matmul_amd

runs ``build.py`` (hipcc for ``libwindow_matmul_hip.so``, g++ for ``window_matmul_kernel.so``)
and installs both next to the package, so that ``import window_matmul`` works without
touching ``sys.path``.  The extension finds the HIP library through ``$ORIGIN``.
"""
import os
import shutil
import sys

from setuptools import Extension, setup
from setuptools.command.build_ext import build_ext

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)


class BuildNative(build_ext):
    """Builds both shared objects in-tree with build.py and copies them into the build tree."""

    def run(self):
        import build as native_build  # build.py next to this file

        # WM_PREBUILT=1 packages the shared objects that are already in the tree (a machine without
        # hipcc, or a test that must not compile); otherwise stale or missing ones are rebuilt
        if os.environ.get("WM_PREBUILT") == "1":
            for name in ("window_matmul_kernel.so", "libwindow_matmul_hip.so"):
                if not os.path.exists(os.path.join(HERE, name)):
                    raise RuntimeError(f"WM_PREBUILT=1 but {name} is not built; run python build.py")
        else:
            native_build.build_all(force=False)
        for name in ("window_matmul_kernel.so", "libwindow_matmul_hip.so"):
            target = os.path.join(self.build_lib, name)
            os.makedirs(os.path.dirname(target) or ".", exist_ok=True)
            shutil.copyfile(os.path.join(HERE, name), target)

    def get_outputs(self):
        return [os.path.join(self.build_lib, n) for n in ("window_matmul_kernel.so", "libwindow_matmul_hip.so")]


setup(
    name="window_matmul",
    version="0.1.0",
    description="Banded matmuls, band softmax and fused window attention for MI355X (gfx950)",
    packages=["window_matmul"],
    py_modules=["wm_ctypes"],
    # a placeholder so that setuptools runs build_ext; the real work is in BuildNative
    ext_modules=[Extension("window_matmul_kernel", sources=[])],
    cmdclass={"build_ext": BuildNative},
    python_requires=">=3.8",
    zip_safe=False,
)
