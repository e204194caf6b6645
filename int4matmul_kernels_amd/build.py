"""Builds the two in-tree binaries of the package:

* ``libint4mm_hip.so`` -- the C-ABI library (include/int4mm.h): hand-written HIP
  kernels compiled by hipcc for gfx950 only.  No torch dependency.
* ``int4matmul.*.so`` -- the Python extension module ``int4matmul`` with the
  reference's eleven entry points (int4matmul.cpp:65-82), compiled by the host
  C++ compiler against torch/pybind11 and linked to the library above.

Run ``python -m int4matmul_kernels_amd.build`` (or ``__graft_entry__.build()``).
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(PKG, "build")
LIB = os.path.join(PKG, "libint4mm_hip.so")
HIP_SOURCES = ["api.hip", "utils.hip", "matvec.hip", "matmul.hip", "skinny.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

HIP_FLAGS = [
    "-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC", "-fvisibility=hidden",
    "-fgpu-rdc" if False else "-fno-gpu-rdc",
    # packed-FP32 VALU ops are switched off for every device compile
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first dwords of a kernel's explicit arguments arrive in registers with the wave (scalar leading arguments
    # only: a record passed by value is still fetched by the wave itself)
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), r.stdout))
    return r.stdout


def build_hip_library(verbose: bool = False) -> str:
    os.makedirs(OBJ, exist_ok=True)
    objs = [os.path.join(OBJ, s.replace(".hip", ".o")) for s in HIP_SOURCES]

    def one(pair):
        src, obj = pair
        return _run([HIPCC, *HIP_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=4) as ex:
        outs = list(ex.map(one, zip(HIP_SOURCES, objs)))
    if verbose:
        print("".join(outs))
    _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB, *objs])
    return LIB


def extension_path() -> str:
    return os.path.join(PKG, "int4matmul" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_extension(verbose: bool = False) -> str:
    """Host-only compile of the pybind11 module; the kernels stay in the C-ABI
    library, so no HIP source passes through torch's build helpers."""
    import torch
    from torch.utils import cpp_extension

    out = extension_path()
    inc = [f"-I{p}" for p in cpp_extension.include_paths()]
    inc += [f"-I{sysconfig.get_paths()['include']}", "-I/opt/rocm/include",
            f"-I{os.path.join(PKG, '..', 'include')}"]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared",
           "-DTORCH_EXTENSION_NAME=int4matmul", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={abi}", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           *inc, os.path.join(CSRC, "binding.cpp"), "-o", out,
           "-Wl,--no-as-needed", f"-L{PKG}", "-lint4mm_hip", "-Wl,--as-needed", f"-L{torch_lib}", "-lc10", "-lc10_hip", "-ltorch",
           "-ltorch_cpu", "-ltorch_hip", "-ltorch_python",
           "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}", "-Wno-attributes"]
    log = _run(cmd)
    if verbose:
        print(log)
    return out


def build_all(verbose: bool = False):
    lib = build_hip_library(verbose)
    ext = build_extension(verbose)
    return lib, ext


if __name__ == "__main__":
    print("\n".join(build_all(verbose="-v" in sys.argv)))
