"""Builds the native pieces in-tree for gfx950.

* ``lib/libfgms_hip.so``  -- the HIP kernels and the C ABI (``include/fgms.h``),
  compiled with hipcc alone; no torch types cross that boundary.
* ``FGMS/backend*.so``    -- the pybind11 torch extension that keeps the
  reference's python surface (``backend/pybind_cuda.cpp:7-11``); it is written
  against HIP directly, so it is compiled with hipcc as well instead of going
  through torch's CUDA-to-HIP source translation.
"""
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "fgms_amd", "csrc")
LIB_DIR = os.path.join(ROOT, "fgms_amd", "lib")
LIB_PATH = os.path.join(LIB_DIR, "libfgms_hip.so")
OBJ_DIR = os.path.join(ROOT, "build", "obj")

HIP_SOURCES = ["fgms_api.hip", "fgms_generic.hip", "fgms_plan.hip", "fgms_mfma.hip", "fgms_small.hip", "fgms_wgrad.hip",
               "fgms_probe.hip", "fgms_kmap.hip", "fgms_wide.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
CXX = os.environ.get("CXX", "g++")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + r.stdout + "\n")
        raise RuntimeError("build step failed: " + cmd[0])
    return r.stdout


def build_hip_lib(verbose=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = []

    def compile_one(src):
        obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
        out = _run([HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(compile_one, HIP_SOURCES))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs)
    return LIB_PATH


def torch_ext_path():
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(ROOT, "FGMS", "backend" + suffix)


def build_torch_ext(verbose=False):
    """FGMS.backend: pybind11 module over the C ABI, linked against torch."""
    import pybind11
    import torch
    from torch.utils import cpp_extension as ce

    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    out = torch_ext_path()
    inc = []
    for p in ce.include_paths() + [pybind11.get_include(), sysconfig.get_paths()["include"],
                                   os.path.join(ROOT, "include")]:
        inc += ["-I", p]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    # host-only translation unit: no device code, so the plain C++ driver does
    cmd = [CXX, "-O2", "-fPIC", "-std=c++17", "-shared",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=backend",
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % abi,
           "-Wno-deprecated-declarations", "-I", "/opt/rocm/include"] + inc + [
           os.path.join(CSRC, "fgms_torch.cpp"), "-o", out,
           "-L", tlib, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
           "-L", LIB_DIR, "-lfgms_hip",
           "-Wl,-rpath,$ORIGIN/../fgms_amd/lib", "-Wl,-rpath," + tlib]
    o = _run(cmd)
    if verbose and o.strip():
        print(o)
    return out


DEMO_PATH = os.path.join(LIB_DIR, "cabi_demo")


def build_cabi_demo(verbose=False):
    """tests/cabi_demo.c: a plain C program over include/fgms.h (host code only)."""
    cmd = [os.environ.get("CC", "gcc"), "-O2", "-std=c11", "-D__HIP_PLATFORM_AMD__=1",
           "-I", "/opt/rocm/include", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "cabi_demo.c"), "-o", DEMO_PATH,
           "-L", LIB_DIR, "-lfgms_hip", "-L", "/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"]
    o = _run(cmd)
    if verbose and o.strip():
        print(o)
    return DEMO_PATH


def up_to_date():
    """True when both shared objects exist and are newer than every source and header."""
    outs = [LIB_PATH, torch_ext_path()]
    if not all(os.path.exists(o) for o in outs):
        return False
    srcs = [os.path.join(CSRC, f) for f in os.listdir(CSRC)] + \
           [os.path.join(ROOT, "include", f) for f in os.listdir(os.path.join(ROOT, "include"))]
    return min(os.path.getmtime(o) for o in outs) >= max(os.path.getmtime(f) for f in srcs)


def build_all(verbose=False, force=True):
    """force=False: keep in-tree products that are newer than all sources."""
    if not force and up_to_date():
        return
    build_hip_lib(verbose)
    build_torch_ext(verbose)
    build_cabi_demo(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
    print("built", LIB_PATH, torch_ext_path())
