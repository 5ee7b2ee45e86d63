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


def _flags():
    return ["-O2", "-std=c++17", "-fPIC", "-Wno-deprecated-declarations",
            "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=" + NAME,
            "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
            "-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include", "-I" + sysconfig.get_paths()["include"]] + \
           ["-I" + p for p in ce.include_paths()]


def _objects():
    return [(os.path.join(HERE, NAME + ".cpp"), os.path.join(HERE, NAME + ".o")),
            (os.path.join(HERE, "example_third_party_compressor.cpp"), os.path.join(HERE, "example_third_party_compressor.o"))]


def compile_objects():
    """The two sources to objects, side by side (each is a minute of torch headers); needs no libplanmoe_hip.so yet."""
    procs = [subprocess.Popen(["g++"] + _flags() + ["-c", src, "-o", obj]) for src, obj in _objects()]
    codes = [p.wait() for p in procs]
    if any(codes):
        raise subprocess.CalledProcessError(max(codes), "g++ -c (extension objects)")


def link():
    csrc = os.path.join(ROOT, "planmoe_amd", "csrc")
    (_, module_obj), (_, example_obj) = _objects()
    libs = ["-L" + p for p in ce.library_paths()] + ["-L/opt/rocm/lib", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip",
            "-ltorch", "-ltorch_python", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"] + ["-Wl,-rpath," + p for p in ce.library_paths()]
    subprocess.check_call(["g++", "-shared", module_obj, "-o", target(), "-L" + csrc, "-lplanmoe_hip", "-Wl,-rpath," + csrc] + libs)
    # the example plug-in: a compressor compiled against include/planmoe/compressor/abstract.h with the
    # same flags and linked against the module just built
    subprocess.check_call(["g++", "-shared", example_obj, "-o", example_target(), target(), "-Wl,-rpath," + HERE] + libs)
    for _, obj in _objects():
        os.remove(obj)
    return target()


def build():
    compile_objects()
    return link()


def example_target():
    return os.path.join(HERE, "libexample_third_party_compressor.so")


if __name__ == "__main__":
    # no argument: everything; --compile / --link: the two halves (the first needs no libplanmoe_hip.so, so
    # __graft_entry__.build() runs it beside the library's own build)
    if sys.argv[1:] == ["--compile"]:
        compile_objects()
    elif sys.argv[1:] == ["--link"]:
        print(link())
    else:
        print(build())
    sys.exit(0)
