"""Builds moodist_amd/_C*.so (the pybind11 module on PyTorch-ROCm) in-tree with g++.

The module contains no device code: it describes torch tensors to libmoodist.so and passes the
current HIP stream, so it is compiled as host C++ against torch's own headers (which carry the
pybind11 that torch itself was built with).
"""

import os
import subprocess
import sys
import sysconfig

import torch
from torch.utils import cpp_extension

here = os.path.dirname(os.path.abspath(__file__))
pkg = os.path.abspath(os.path.join(here, "..", ".."))
root = os.path.abspath(os.path.join(pkg, ".."))
out = os.path.join(pkg, "_C" + sysconfig.get_config_var("EXT_SUFFIX"))

inc = cpp_extension.include_paths() + [sysconfig.get_paths()["include"], os.path.join(root, "include"),
                                       "/opt/rocm/include"]
libdir = os.path.join(os.path.dirname(torch.__file__), "lib")
cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++20", "-fPIC", "-shared", "-fvisibility=hidden",
       "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), "-D__HIP_PLATFORM_AMD__=1",
       "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_C", "-Wno-deprecated-declarations"]
# the build magic of the core this module is built together with (build_host.sh draws it)
if os.environ.get("MOODIST_BUILD_MAGIC"):
    cmd.append("-DMOODIST_BUILD_MAGIC=" + os.environ["MOODIST_BUILD_MAGIC"])
cmd += ["-I" + p for p in inc]
cmd += [os.path.join(here, "module.cc"), "-o", out, "-L" + libdir, "-Wl,-rpath," + libdir,
        "-ltorch_python", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip", "-ldl"]
print(" ".join(cmd))
if len(sys.argv) > 1:  # another output path (a test builds a module of another magic)
    out = sys.argv[1]
    cmd[cmd.index("-o") + 1] = out
subprocess.check_call(cmd)
print("built", out)
