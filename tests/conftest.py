import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tt-metal_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import bfp_oracle

    bfp_oracle.build()
    return bfp_oracle


# knobs of libttmi's test entry point (tt-metal_amd/csrc/ttmi_internal.h: TTMI_KNOB_*)
KNOB = {"kernel": 0, "workgroups": 1, "block": 2, "spin_limit": 3, "drop_partial_sums": 4, "xcds": 5}
KERNEL_CODE = {"stream": 1, "wide": 2, "tile": 3, "expanded": 4}


@pytest.fixture
def test_library():
    """The test runs on libttmi_test.so / _ttmi_test: the product sources built with -DTTMI_TEST_HOOKS, which adds the
    ttmi_test_* entry points (the product library has none of them)."""
    import tt_lib.tensor

    tt_lib.tensor.use_test_library(True)
    try:
        from ttmi import capi

        yield capi.lib()
    finally:
        tt_lib.tensor.use_test_library(False)


@pytest.fixture
def knobs(test_library):
    """knobs(name, value) on the library's test entry point (name: kernel = stream | wide | tile | expanded, workgroups,
    block = 256 | 128 | 4 | 384, spin_limit, drop_partial_sums, xcds = 1 | 8); everything set is cleared again after the test."""
    import ctypes

    from ttmi import capi

    L = test_library
    L.ttmi_test_set_knob.restype = ctypes.c_int
    L.ttmi_test_set_knob.argtypes = [ctypes.c_int, ctypes.c_uint32, ctypes.c_int]
    touched = []

    def set_knob(name, value):
        which = KNOB[name]
        capi.check(L.ttmi_test_set_knob(which, KERNEL_CODE[value] if name == "kernel" else int(value), 1))
        touched.append(which)

    yield set_knob
    for which in touched:
        L.ttmi_test_set_knob(which, 0, 0)
