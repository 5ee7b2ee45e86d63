"""Loader of the torch C++ extension that carries the reference's pybind surface
(``schemoe_custom_kernel``: compress_operation / comm_operation / decompress_operation /
clear_ptr_lst, and ``torch.ops.tutel_ops.cumsum``) on top of libplanmoe_hip.

    from planmoe_amd import ext
    ck = ext.load()                 # the module
    ext.install_alias()             # makes ``import schemoe_custom_kernel`` resolve to it
"""
import importlib.util
import os
import sys
import sysconfig

import torch

from . import _lib  # noqa: F401  (loads libplanmoe_hip.so first; raises if it is missing)

_HERE = os.path.dirname(os.path.abspath(__file__))
NAME = "schemoe_custom_kernel"
PATH = os.path.join(_HERE, "csrc", "ext", NAME + sysconfig.get_config_var("EXT_SUFFIX"))
_module = None


def load():
    global _module
    if _module is None:
        if not os.path.exists(PATH):
            raise ImportError("planmoe_amd: %s is missing; build it with "
                              "python planmoe_amd/csrc/ext/build.py (or __graft_entry__.build())" % PATH)
        spec = importlib.util.spec_from_file_location(NAME, PATH)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        torch.ops.load_library(PATH)          # registers tutel_ops::cumsum (jit_kernels/gating.py:9)
        _module = mod
    return _module


def install_alias():
    sys.modules[NAME] = load()
    return sys.modules[NAME]
