"""Builds the torch extension grokking_optimizers/_ops*.so from ops_shim.cpp and ops_bilevel.cpp.

Plain g++ against the installed torch headers (no hipify step, no JIT cache):
the shim contains no device code, it only forwards to libsg_hip.so, which it
finds at run time through an $ORIGIN-relative rpath.
"""
import os
import subprocess
import sys
import sysconfig

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)


def main():
    tdir = os.path.dirname(torch.__file__)
    ext = sysconfig.get_config_var("EXT_SUFFIX")
    out = os.path.join(PKG, "grokking_optimizers", "_ops" + ext)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
           "-DTORCH_EXTENSION_NAME=_ops", "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=1",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-I" + os.path.join(tdir, "include"), "-I" + os.path.join(tdir, "include", "torch", "csrc", "api", "include"),
           "-I" + sysconfig.get_paths()["include"], "-I" + os.path.join(rocm, "include"),
           os.path.join(HERE, "ops_shim.cpp"), os.path.join(HERE, "ops_bilevel.cpp"), "-o", out,
           "-L" + tdir + "/lib", "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lc10_hip", "-ltorch_hip",
           "-L" + os.path.join(PKG, "lib"), "-lsg_hip",
           "-Wl,-rpath,$ORIGIN/../lib", "-Wl,-rpath," + tdir + "/lib", "-Wno-unused-variable"]
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    print("built", out)


if __name__ == "__main__":
    sys.exit(main())
