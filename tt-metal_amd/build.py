"""Builds libttmi.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python tt-metal_amd/build.py            # rebuild what is out of date
    python tt-metal_amd/build.py --force
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


def _compile(src: str, verbose: bool) -> None:
    path = os.path.join(CSRC, src)
    obj = os.path.join(LIB_DIR, src.replace(".hip", ".o"))
    if src in ISA_CHECKED:
        # the device assembly of this file is inspected before the object is built (see check_isa.py)
        asm = os.path.join(LIB_DIR, src.replace(".hip", ".s"))
        cmd = [HIPCC] + FLAGS + ["-S", "--cuda-device-only", path, "-o", asm]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
        import check_isa
        if getattr(check_isa, ISA_CHECKED[src])(asm):
            if os.path.exists(obj):
                os.remove(obj)
            raise RuntimeError(f"{src}: the compiler moved registers of hand-scheduled loads; see check_isa.py")
        os.remove(asm)
    cmd = [HIPCC] + FLAGS + ["-c", path, "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def build(force: bool = False, verbose: bool = False) -> str:
    from concurrent.futures import ThreadPoolExecutor

    os.makedirs(LIB_DIR, exist_ok=True)
    objs = [os.path.join(LIB_DIR, src.replace(".hip", ".o")) for src in SOURCES]
    stale = [src for src, obj in zip(SOURCES, objs) if force or _stale(obj, [os.path.join(CSRC, src)] + HEADERS)]
    # the translation units are independent: compile those that are out of date side by side
    with ThreadPoolExecutor(max_workers=min(4, max(1, len(stale)))) as pool:
        list(pool.map(lambda src: _compile(src, verbose), stale))
    if force or _stale(LIB, objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
    return LIB


def build_bindings(force: bool = False, verbose: bool = False) -> str:
    """Builds the pybind11 module tt-metal_amd/lib/_ttmi*.so: the host layer (csrc/host/tensor_ops.cpp: Tensor, validation,
    conversion sequences, dispatch) and the bindings, host C++ only; links libttmi.so next to it and the HIP runtime."""
    import sysconfig

    import pybind11

    build(force=False, verbose=verbose)
    sources = [os.path.join(CSRC, "ttmi_pybind.cpp"), os.path.join(CSRC, "host", "tensor_ops.cpp")]
    deps = sources + [os.path.join(CSRC, "host", "tensor_ops.hpp"), os.path.join(ROOT, "include", "ttmi.h"), LIB]
    out = os.path.join(LIB_DIR, "_ttmi" + sysconfig.get_config_var("EXT_SUFFIX"))
    if force or _stale(out, deps):
        rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
        cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-shared", "-fPIC", "-fvisibility=hidden", "-D__HIP_PLATFORM_AMD__",
               "-I", pybind11.get_include(), "-I", sysconfig.get_paths()["include"], "-I", os.path.join(ROOT, "include"), "-I", CSRC,
               "-I", os.path.join(rocm, "include")] + sources + [
               "-o", out, "-L", LIB_DIR, "-lttmi", "-L", os.path.join(rocm, "lib"), "-lamdhip64", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(rocm, "lib")]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
    return out


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
    print(build_bindings(force="--force" in sys.argv, verbose=True))
