"""Loader of the pybind11 module `_ttmi` (tt-metal_amd/csrc/ttmi_pybind.cpp), built in-tree by build.py."""
from __future__ import annotations

import glob
import importlib.util
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_DIR = os.path.join(os.path.dirname(_HERE), "lib")
_mod = None


def module():
    """Returns the loaded extension module; raises RuntimeError when it has not been built."""
    global _mod
    if _mod is None:
        found = sorted(glob.glob(os.path.join(_LIB_DIR, "_ttmi*.so")))
        if not found:
            raise RuntimeError(f"pybind11 module _ttmi not built in {_LIB_DIR} (run `python tt-metal_amd/build.py`)")
        spec = importlib.util.spec_from_file_location("_ttmi", found[0])
        _mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(_mod)
    return _mod
