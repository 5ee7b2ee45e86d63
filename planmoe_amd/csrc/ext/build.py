"""Builds schemoe_custom_kernel*.so (the reference's pybind module name) in planmoe_amd/csrc/ext with
g++ against torch's headers and libplanmoe_hip.so.  Run by __graft_entry__.build()."""
import os
import subprocess
import sys
import sysconfig

import torch
from torch.utils import cpp_extension as ce

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.abspath(os.path.join(HERE, "..", "..", ".."))
NAME = "schemoe_custom_kernel"


def target():
    return os.path.join(HERE, NAME + sysconfig.get_config_var("EXT_SUFFIX"))


def build():
    csrc = os.path.join(ROOT, "planmoe_amd", "csrc")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wno-deprecated-declarations",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=" + NAME,
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include", "-I" + sysconfig.get_paths()["include"]]
    cmd += ["-I" + p for p in ce.include_paths()]
    cmd += [os.path.join(HERE, NAME + ".cpp"), "-o", target()]
    cmd += ["-L" + p for p in ce.library_paths()] + ["-L" + csrc, "-L/opt/rocm/lib"]
    cmd += ["-lplanmoe_hip", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python", "-lamdhip64",
            "-Wl,-rpath," + csrc, "-Wl,-rpath,/opt/rocm/lib"] + ["-Wl,-rpath," + p for p in ce.library_paths()]
    subprocess.check_call(cmd)
    # the example plug-in: a compressor compiled against include/planmoe/compressor/abstract.h with the
    # same flags and linked against the module just built
    flags = cmd[1:cmd.index(os.path.join(HERE, NAME + ".cpp"))]
    libs = [a for a in cmd[cmd.index(target()) + 1:] if a != "-lplanmoe_hip"]
    subprocess.check_call(["g++"] + flags + [os.path.join(HERE, "example_third_party_compressor.cpp"), "-o", example_target(),
                                             target(), "-Wl,-rpath," + HERE] + libs)
    return target()


def example_target():
    return os.path.join(HERE, "libexample_third_party_compressor.so")


if __name__ == "__main__":
    print(build())
    sys.exit(0)
