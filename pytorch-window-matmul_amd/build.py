"""In-tree build of the two native artefacts, for gfx950 only.

* ``libwindow_matmul_hip.so`` -- the C-ABI library (HIP kernels + launchers),
  compiled with hipcc from ``csrc/*.hip``.  It depends on the HIP runtime only.
* ``window_matmul_kernel.so`` -- the PyTorch-ROCm extension module the Python
  package imports, compiled with g++ from ``csrc/binding.cpp`` and linked
  against the library above (found at run time through ``$ORIGIN``).

Both land next to this file so that putting this directory on ``sys.path``
makes ``import window_matmul`` and ``import window_matmul_kernel`` work.
Run ``python build.py`` (add ``--force`` to rebuild up-to-date targets).
"""
import glob
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
HIP_LIB = os.path.join(HERE, "libwindow_matmul_hip.so")
EXT_LIB = os.path.join(HERE, "window_matmul_kernel.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # extra hipcc flags for experiments, e.g. WM_EXTRA_FLAGS=-DWM_VECTOR_MAX_W=0
    *os.environ.get("WM_EXTRA_FLAGS", "").split(),
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _newer(target, sources):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(s) <= t for s in sources)


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if out.strip():
        print(out, flush=True)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}")


def build_hip_library(force=False):
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    deps = sources + glob.glob(os.path.join(CSRC, "*.hpp")) + glob.glob(os.path.join(INCLUDE, "*.h"))
    if not force and _newer(HIP_LIB, deps):
        return HIP_LIB
    objs = []
    procs = []
    headers = [d for d in deps if d not in sources]
    for src in sources:
        obj = os.path.join(CSRC, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        if not force and _newer(obj, [src] + headers):
            continue  # this object is still current: only stale translation units are recompiled
        cmd = [os.path.join(ROCM, "bin", "hipcc"), *HIPCC_FLAGS, "-c", src, "-o", obj]
        print("+", " ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for cmd, proc in procs:
        out, _ = proc.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if out.strip():
            print(out, flush=True)
        if proc.returncode != 0:
            raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}")
    _run([os.path.join(ROCM, "bin", "hipcc"), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", HIP_LIB])
    return HIP_LIB


def build_extension(force=False):
    import torch

    src = os.path.join(CSRC, "binding.cpp")
    deps = [src, HIP_LIB] + glob.glob(os.path.join(INCLUDE, "*.h"))
    if not force and _newer(EXT_LIB, deps):
        return EXT_LIB
    tdir = os.path.dirname(torch.__file__)
    cmd = [
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
        "-DTORCH_EXTENSION_NAME=window_matmul_kernel", "-DTORCH_API_INCLUDE_EXTENSION_H",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DHIPBLAS_V2",
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        f"-I{tdir}/include", f"-I{tdir}/include/torch/csrc/api/include",
        f"-I{ROCM}/include", f"-I{sysconfig.get_paths()['include']}",
        src,
        f"-L{HERE}", "-lwindow_matmul_hip", "-Wl,-rpath,$ORIGIN",
        f"-L{tdir}/lib", f"-Wl,-rpath,{tdir}/lib",
        "-ltorch_python", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
        "-o", EXT_LIB,
    ]
    _run(cmd)
    return EXT_LIB


def build_all(force=False):
    build_hip_library(force)
    build_extension(force)


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
