"""The C-ABI library loads and exports every symbol include/ttmi.h declares (no compute, no GPU)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ttmi.h")).read()
    return sorted(set(re.findall(r"TTMI_API[^;(]*?\b(ttmi_\w+)\s*\(", text)))


def test_header_symbols_are_exported():
    from ttmi import capi

    if not os.path.exists(capi.LIB_PATH):
        pytest.skip("libttmi.so not built in this checkout (python tt-metal_amd/build.py)")
    names = declared_symbols()
    assert len(names) >= 12
    assert sorted(capi.SYMBOLS) == names
    L = ctypes.CDLL(capi.LIB_PATH)
    for n in names:
        assert hasattr(L, n), n


def test_size_helpers_need_no_gpu():
    from ttmi import capi

    if not os.path.exists(capi.LIB_PATH):
        pytest.skip("libttmi.so not built")
    L = capi.lib()
    # tt_backend_api_types.hpp:109-132
    assert [L.ttmi_tile_size(d) for d in (3, 4, 0, 1, 2, 6, 5)] == [1088, 576, 2048, 4096, 4096, 2048, 0]
    assert L.ttmi_tiled_size_bytes(3, 1, 1024, 1024) == 1114112
    assert L.ttmi_tiled_size_bytes(4, 1, 4096, 4096) == 9437184
    assert L.ttmi_tiled_size_bytes(3, 6, 7, 3) == 6 * 1088


def test_matmul_workspace_sizes_follow_the_decomposition(monkeypatch):
    """What a caller has to bring for a GEMM of its own stream: 16 KB of partial-sum slots per computing workgroup of the
    128-column kernel (one band of rows), nothing when every output has a workgroup of its own, the expanded weights
    (2 bytes each) from 512 rows on."""
    from ttmi import capi

    if not os.path.exists(capi.LIB_PATH):
        pytest.skip("libttmi.so not built")
    for name in ("TTMI_MATMUL_KERNEL", "TTMI_MATMUL_WGS", "TTMI_MATMUL_BM"):
        monkeypatch.delenv(name, raising=False)
    ws = capi.lib().ttmi_matmul_bfp_workspace_bytes
    assert ws(1, 32, 4544, 18176, 3) == 142 * 3 * 16384        # 142 groups of 128 columns, 512 // 143 = 3 k ranges each
    assert ws(1, 32, 18176, 4544, 3) == 36 * 7 * 16384         # 36 groups (the last one half empty), 256 // 36 = 7
    assert ws(1, 32, 64, 4096, 3) == 0                         # 2 k-tiles: never shared
    assert ws(1, 64, 4544, 18176, 3) == 0                      # two bands, 64-column kernel: 568 groups fill the chip
    assert ws(1, 256, 4096, 4096, 3) == 0                      # fused tiled kernels
    assert ws(1, 2048, 4096, 14336, 3) == 4096 * 14336 * 2     # expanded weights
    assert ws(0, 32, 64, 64, 3) == 0


def test_argument_validation_returns_errors_without_launching():
    from ttmi import capi

    if not os.path.exists(capi.LIB_PATH):
        pytest.skip("libttmi.so not built")
    L = capi.lib()
    assert L.ttmi_pack_fp32_vec_as_bfp_tiles(0, None, 1, 0, None, None) == 1
    assert b"BFLOAT8_B" in L.ttmi_last_error()
    assert L.ttmi_pack_fp32_vec_as_bfp_tiles(3, None, 1, 0, None, None) == 1
    assert L.ttmi_tilize(None, 3, 1, 32, 32, None, None) == 1
    one = ctypes.c_void_p(16)
    # K, N must be tile multiples; weight batch 1 or batch
    assert L.ttmi_matmul_bfp(one, 0, one, 3, 1, 1, 32, 33, 64, None, 0, one, 0, 0, None, 0, None) == 1
    assert b"multiples of 32" in L.ttmi_last_error()
    assert L.ttmi_matmul_bfp(one, 0, one, 3, 4, 2, 32, 32, 64, None, 0, one, 0, 0, None, 0, None) == 1
    assert L.ttmi_matmul_bfp(one, 1, one, 3, 1, 1, 7, 32, 64, None, 0, one, 0, 0, None, 0, None) == 1
    assert L.ttmi_matmul_bfp(one, 0, one, 2, 1, 1, 32, 32, 64, None, 0, one, 0, 0, None, 0, None) == 1


def test_missing_library_fails_loudly(monkeypatch):
    from ttmi import capi

    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", "/nonexistent/libttmi.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        capi.lib()
