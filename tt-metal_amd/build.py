"""Builds libttmi.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree, and the pybind11 module _ttmi over it.

    python tt-metal_amd/build.py            # rebuild what is out of date
    python tt-metal_amd/build.py --force

Next to them a test build of both: libttmi_test.so is the same sources with -DTTMI_TEST_HOOKS, which adds the entry points
ttmi_test_* (forcing a kernel, a decomposition, a give-up; reading the host's index functions) that the product library
does not have, and _ttmi_test is the same bindings over it.  Only tests load those two.
"""
from __future__ import annotations

import os
import subprocess
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libttmi.so")
LIB_TEST = os.path.join(LIB_DIR, "libttmi_test.so")
# translation units that the test hooks change (they are compiled twice); the others are shared by the two libraries
HOOKED = ["host_state.hip", "bfp_matmul.hip", "bfp_matmul_tile.hip"]
SOURCES = ["ttmi_capi.hip", "host_state.hip", "bfp_codec.hip", "bfp_matmul.hip", "bfp_matmul_tile.hip", "bfp_matmul_expanded.hip", "eltwise.hip"]
# files whose device assembly is inspected before the object is built, and the check of check_isa.py that applies
ISA_CHECKED = {"bfp_matmul.hip": "check", "bfp_matmul_tile.hip": "check_ring_operands"}
HEADERS = [os.path.join(CSRC, "ttmi_internal.h"), os.path.join(CSRC, "bfp_dequant.h"), os.path.join(ROOT, "include", "ttmi.h")]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # packed fp32 VALU forms have produced wrong results on this hardware pool: keep the compiler off them
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


def _stale(target: str, deps) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _object(src: str, hooks: bool) -> str:
    return os.path.join(LIB_DIR, src.replace(".hip", "_test.o" if hooks else ".o"))


def _compile(src: str, hooks: bool, verbose: bool) -> None:
    path = os.path.join(CSRC, src)
    obj = _object(src, hooks)
    flags = FLAGS + (["-DTTMI_TEST_HOOKS"] if hooks else [])
    if src in ISA_CHECKED:
        # the device assembly of this file is inspected before the object is built (see check_isa.py)
        asm = obj[:-2] + ".s"
        cmd = [HIPCC] + flags + ["-S", "--cuda-device-only", path, "-o", asm]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
        import check_isa
        if getattr(check_isa, ISA_CHECKED[src])(asm):
            if os.path.exists(obj):
                os.remove(obj)
            raise RuntimeError(f"{src}: the compiler moved registers of hand-scheduled loads; see check_isa.py")
        os.remove(asm)
    cmd = [HIPCC] + flags + ["-c", path, "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def build(force: bool = False, verbose: bool = False) -> str:
    from concurrent.futures import ThreadPoolExecutor

    os.makedirs(LIB_DIR, exist_ok=True)
    jobs = [(src, False) for src in SOURCES] + [(src, True) for src in HOOKED]
    stale = [(src, hooks) for src, hooks in jobs if force or _stale(_object(src, hooks), [os.path.join(CSRC, src)] + HEADERS)]
    # the translation units are independent: compile those that are out of date side by side
    with ThreadPoolExecutor(max_workers=min(5, max(1, len(stale)))) as pool:
        list(pool.map(lambda job: _compile(job[0], job[1], verbose), stale))
    for lib, hooks in ((LIB, False), (LIB_TEST, True)):
        objs = [_object(src, hooks and src in HOOKED) for src in SOURCES]
        if force or _stale(lib, objs):
            cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs
            if verbose:
                print(" ".join(cmd), flush=True)
            subprocess.run(cmd, check=True)
    return LIB


def build_bindings(force: bool = False, verbose: bool = False) -> str:
    """Builds the pybind11 module tt-metal_amd/lib/_ttmi*.so: the host layer (csrc/host/tensor_ops.cpp: Tensor, validation,
    conversion sequences, dispatch) and the bindings, host C++ only; links libttmi.so next to it and the HIP runtime.
    And _ttmi_test*.so, the same over libttmi_test.so."""
    import sysconfig

    import pybind11

    build(force=False, verbose=verbose)
    sources = [os.path.join(CSRC, "ttmi_pybind.cpp"), os.path.join(CSRC, "host", "tensor_ops.cpp")]
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    first = None
    for name, lib_name, lib_path in (("_ttmi", "ttmi", LIB), ("_ttmi_test", "ttmi_test", LIB_TEST)):
        deps = sources + [os.path.join(CSRC, "host", "tensor_ops.hpp"), os.path.join(ROOT, "include", "ttmi.h"), lib_path]
        out = os.path.join(LIB_DIR, name + sysconfig.get_config_var("EXT_SUFFIX"))
        first = first or out
        if force or _stale(out, deps):
            cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-shared", "-fPIC", "-fvisibility=hidden", "-D__HIP_PLATFORM_AMD__",
                   "-DTTMI_PYBIND_NAME=" + name,
                   "-I", pybind11.get_include(), "-I", sysconfig.get_paths()["include"], "-I", os.path.join(ROOT, "include"), "-I", CSRC,
                   "-I", os.path.join(rocm, "include")] + sources + [
                   "-o", out, "-L", LIB_DIR, "-l" + lib_name, "-L", os.path.join(rocm, "lib"), "-lamdhip64", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(rocm, "lib")]
            if verbose:
                print(" ".join(cmd), flush=True)
            subprocess.run(cmd, check=True)
    return first


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
    print(build_bindings(force="--force" in sys.argv, verbose=True))
