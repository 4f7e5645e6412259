"""Loader of the pybind11 module `_ttmi` (tt-metal_amd/csrc/ttmi_pybind.cpp), built in-tree by build.py."""
from __future__ import annotations

import glob
import importlib.util
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_DIR = os.path.join(os.path.dirname(_HERE), "lib")
_mods = {}


def module(name: str = "_ttmi"):
    """Returns the loaded extension module; raises RuntimeError when it has not been built.  `_ttmi_test` is the same
    bindings over libttmi_test.so (the library with the test hooks): tests only."""
    if name not in _mods:
        found = sorted(glob.glob(os.path.join(_LIB_DIR, name + ".*.so")))
        if not found:
            raise RuntimeError(f"pybind11 module {name} not built in {_LIB_DIR} (run `python tt-metal_amd/build.py`)")
        spec = importlib.util.spec_from_file_location(name, found[0])
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _mods[name] = mod
    return _mods[name]
