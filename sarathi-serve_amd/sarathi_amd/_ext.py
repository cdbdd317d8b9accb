"""Loads the compiled extension (``_C.so``) that sits next to this file.

The extension is built in-tree by ``build.py`` one directory up; it links
against ``lib/libsarathi_ops_hip.so`` (the C ABI of include/sarathi_ops.h).
Nothing here falls back to another implementation.
"""
import importlib.machinery
import importlib.util
import os

import torch  # noqa: F401  (must be loaded first: _C.so resolves libtorch and the HIP runtime from it)

_HERE = os.path.dirname(os.path.abspath(__file__))
EXT_PATH = os.path.join(_HERE, "_C.so")
ABI_LIB_PATH = os.path.join(_HERE, "lib", "libsarathi_ops_hip.so")


def _load():
    for path in (ABI_LIB_PATH, EXT_PATH):
        if not os.path.exists(path):
            raise ImportError(
                "sarathi_amd: %s is missing; build it with `python %s`"
                % (path, os.path.join(os.path.dirname(_HERE), "build.py")))
    loader = importlib.machinery.ExtensionFileLoader(__package__ + "._C", EXT_PATH)
    spec = importlib.util.spec_from_file_location(__package__ + "._C", EXT_PATH, loader=loader)
    module = importlib.util.module_from_spec(spec)
    loader.exec_module(module)
    return module


C = _load()
