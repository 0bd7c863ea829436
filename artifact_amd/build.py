"""Compile librof.so (gfx950 kernels + host code) in-tree with hipcc / g++.

    python -m artifact_amd.build

hipcc cross-compiles for gfx950 without a GPU.  The library is loaded with ctypes
(artifact_amd/_lib.py) and does not link against PyTorch.  `build_torch_module` then compiles the thin
C++ module `artifact_amd/_ROF*.so` (csrc/rof_torch.cpp: upstream's seven `ROF` operators over the C ABI),
which links against PyTorch and librof.so.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "librof.so")

HOST_SOURCES = ["plan_builder.cpp", "hub_patterns.cpp", "dynamic_greedy.cpp", "layout.cpp"]
HIP_SOURCES = ["agg_kernels.hip", "agg_rows_f32_partial.hip", "agg_rows_f32_dst.hip", "agg_cluster_f32.hip", "agg_coop_f32.hip", "agg_coop_bf16.hip",
               "agg_rows_bf16_partial.hip", "agg_rows_bf16_dst.hip", "agg_cluster_bf16.hip"]

# packed fp32 instructions stay off: the compiler must not form v_pk_{add,mul,fma}_f32
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops", "-Wno-unused-command-line-argument"]
HOST_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-fopenmp", "-Wall"]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def build_library(verbose=True):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    gxx = shutil.which("g++") or "g++"
    inc = ["-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    for s in HOST_SOURCES:
        o = os.path.join(objdir, s + ".o")
        _run([gxx] + HOST_FLAGS + inc + ["-c", os.path.join(CSRC, s), "-o", o])
        objs.append(o)
    # the kernel translation units are independent: compile them side by side
    procs = []
    for s in HIP_SOURCES:
        o = os.path.join(objdir, s + ".o")
        cmd = [hipcc] + HIP_FLAGS + inc + ["-c", os.path.join(CSRC, s), "-o", o]
        print("+", " ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd)))
        objs.append(o)
    for cmd, pr in procs:
        if pr.wait() != 0:
            raise subprocess.CalledProcessError(pr.returncode, cmd)
    _run([hipcc, "-shared", "-fPIC", "-o", LIB] + objs + ["-fopenmp", "-lgomp"])
    return LIB


def torch_module_path():
    import sysconfig

    return os.path.join(HERE, "_ROF" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_torch_module():
    """csrc/rof_torch.cpp -> artifact_amd/_ROF<ext suffix>.so with g++ against the installed PyTorch's headers and
    libraries (host code only: the kernels are in librof.so, found at run time next to the module)."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    gxx = shutil.which("g++") or "g++"
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    out = torch_module_path()
    cmd = [gxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-w", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=_ROF", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-I" + os.path.join(ROOT, "include")]
    cmd += ["-I" + p for p in cpp_extension.include_paths()] + ["-I" + os.path.join(rocm, "include"),
                                                                 "-I" + sysconfig.get_paths()["include"]]
    cmd += [os.path.join(CSRC, "rof_torch.cpp"), "-o", out, "-L" + tlib, "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu",
            "-ltorch_hip", "-ltorch_python", "-L" + HERE, "-l:librof.so", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + tlib]
    _run(cmd)
    return out


if __name__ == "__main__":
    build_library()
    print("built", LIB)
    print("built", build_torch_module())
    sys.exit(0)
