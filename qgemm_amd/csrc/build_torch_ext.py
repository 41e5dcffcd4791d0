#!/usr/bin/env python3
"""Builds qgemm_amd/qgemm_python*.so, the torch extension over libqgemm.so, in-tree.

One host-only translation unit (torch_ext.cpp) compiled with hipcc as plain C++ against the headers and
libraries of the torch that runs this script; no JIT cache, no source rewriting."""
import os
import subprocess
import sys
import sysconfig

import torch
from torch.utils import cpp_extension as ext

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)


def main():
    out = os.path.join(PKG, "qgemm_python" + sysconfig.get_config_var("EXT_SUFFIX"))
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "-O2", "-std=c++17", "-fPIC", "-shared", "-w",
           "-x", "c++", os.path.join(HERE, "torch_ext.cpp"),
           "-DTORCH_EXTENSION_NAME=qgemm_python", "-DTORCH_API_INCLUDE_EXTENSION_H", "-D__HIP_PLATFORM_AMD__=1",
           "-DUSE_ROCM=1", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    for inc in ext.include_paths(device_type="cuda") + [sysconfig.get_paths()["include"], "/opt/rocm/include"]:
        cmd += ["-isystem", inc]
    cmd += ["-L" + torch_lib, "-L" + PKG, "-lqgemm", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch",
            "-ltorch_python", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib, "-o", out]
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    print("built", out)


if __name__ == "__main__":
    sys.exit(main())
