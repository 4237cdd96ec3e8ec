#!/usr/bin/env python3
"""Builds flashbias_amd/_fb_torch.so, the operator's autograd function in C++ (fb_torch.cpp), with the
host compiler against the installed torch: no device code, it calls libflashbias_hip.so through the
C ABI (which must have been built first: it is linked by name, found at run time next to the module).
Run by `make torch_ext` and by __graft_entry__.build()."""
import os
import subprocess
import sys
import sysconfig

import torch
from torch.utils import cpp_extension

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
OUT = os.path.join(PKG, "_fb_torch.so")


def main():
    cxx = os.environ.get("CXX", "g++")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unknown-pragmas", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=_fb_torch", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I" + os.path.join(PKG, "..", "include")]
    for inc in cpp_extension.include_paths(True) + [sysconfig.get_paths()["include"], "/opt/rocm/include"]:
        cmd += ["-isystem", inc]
    cmd += [os.path.join(HERE, "fb_torch.cpp"), "-o", OUT]
    for lib in cpp_extension.library_paths(True):
        if os.path.isdir(lib):
            cmd += ["-L" + lib, "-Wl,-rpath," + lib]
    cmd += ["-L" + PKG, "-Wl,-rpath,$ORIGIN", "-lflashbias_hip", "-lc10", "-ltorch_cpu", "-ltorch", "-ltorch_python", "-lc10_hip",
            "-ltorch_hip"]
    print(" ".join(cmd))
    subprocess.check_call(cmd)
    return 0


if __name__ == "__main__":
    sys.exit(main())
