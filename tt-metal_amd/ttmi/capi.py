"""ctypes view of the C ABI in ``include/ttmi.h`` plus thin helpers that pass torch device pointers.

There is no CPU fallback: if ``lib/libttmi.so`` is missing or a call fails, a RuntimeError is raised.
torch is used for device memory and streams only.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libttmi.so")
# the test build of the same sources (-DTTMI_TEST_HOOKS): the product library plus the ttmi_test_* entry points; tests only
LIB_TEST_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libttmi_test.so")

BFLOAT16, FLOAT32, UINT32, BFLOAT8_B, BFLOAT4_B, UINT16 = 0, 1, 2, 3, 4, 6
ROW_MAJOR, TILE = 0, 1
ACT_NONE, ACT_RELU, ACT_GELU, ACT_SILU = 0, 1, 2, 3
OP_ADD, OP_SUB, OP_MUL, OP_RELU, OP_GELU, OP_SILU = 0, 1, 2, 17, 18, 19
TILE_BYTES = {BFLOAT8_B: 1088, BFLOAT4_B: 576, BFLOAT16: 2048, UINT16: 2048, FLOAT32: 4096, UINT32: 4096}

# every symbol include/ttmi.h declares
SYMBOLS = (
    "ttmi_last_error", "ttmi_version", "ttmi_tile_size", "ttmi_tiled_size_bytes",
    "ttmi_pack_fp32_vec_as_bfp_tiles", "ttmi_unpack_bfp_tiles_into_float_vec",
    "ttmi_pack_rowmajor_as_bfp_tiles", "ttmi_unpack_bfp_tiles_as_rowmajor",
    "ttmi_tilize", "ttmi_untilize", "ttmi_matmul_bfp_workspace_bytes", "ttmi_matmul_bfp",
    "ttmi_eltwise_bf16", "ttmi_copy_window", "ttmi_unpad_tiles", "ttmi_typecast_tiles", "ttmi_device_status", "ttmi_matmul_bfp_static",
    "ttmi_matmul_bfp_gated_workspace_bytes", "ttmi_matmul_bfp_gated", "ttmi_matmul_bf16_workspace_bytes", "ttmi_matmul_bf16",
    "ttmi_release_scratch", "ttmi_matmul_bfp_ab_supported", "ttmi_matmul_bfp_ab", "ttmi_matmul_bfp_plan",
)

_lib = None
_loaded = {}


def use_test_library(on: bool) -> None:
    """Tests only: every call below goes to libttmi_test.so (the library with the ttmi_test_* hooks) until switched back."""
    global _lib
    _lib = None
    if on:
        _lib = _load(LIB_TEST_PATH)


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        _lib = _load(LIB_PATH)
    return _lib


def _load(path: str) -> ctypes.CDLL:
    if path not in _loaded:
        if not os.path.exists(path):
            raise RuntimeError(
                f"{path} is not built: run `python tt-metal_amd/build.py` (needs hipcc); there is no CPU fallback"
            )
        L = ctypes.CDLL(path)
        vp, u32, i32, sz = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_int, ctypes.c_size_t
        L.ttmi_last_error.restype = ctypes.c_char_p
        L.ttmi_last_error.argtypes = []
        L.ttmi_version.restype = ctypes.c_char_p
        L.ttmi_version.argtypes = []
        L.ttmi_tile_size.restype = u32
        L.ttmi_tile_size.argtypes = [i32]
        L.ttmi_tiled_size_bytes.restype = sz
        L.ttmi_tiled_size_bytes.argtypes = [i32, u32, u32, u32]
        L.ttmi_pack_fp32_vec_as_bfp_tiles.restype = i32
        L.ttmi_pack_fp32_vec_as_bfp_tiles.argtypes = [i32, vp, sz, i32, vp, vp]
        L.ttmi_unpack_bfp_tiles_into_float_vec.restype = i32
        L.ttmi_unpack_bfp_tiles_into_float_vec.argtypes = [i32, vp, sz, i32, vp, vp]
        L.ttmi_pack_rowmajor_as_bfp_tiles.restype = i32
        L.ttmi_pack_rowmajor_as_bfp_tiles.argtypes = [i32, vp, i32, u32, u32, u32, sz, sz, vp, vp]
        L.ttmi_unpack_bfp_tiles_as_rowmajor.restype = i32
        L.ttmi_unpack_bfp_tiles_as_rowmajor.argtypes = [i32, vp, u32, u32, u32, vp, i32, vp]
        L.ttmi_tilize.restype = i32
        L.ttmi_tilize.argtypes = [vp, u32, u32, u32, u32, vp, vp]
        L.ttmi_untilize.restype = i32
        L.ttmi_untilize.argtypes = [vp, u32, u32, u32, u32, vp, vp]
        L.ttmi_matmul_bfp_workspace_bytes.restype = sz
        L.ttmi_matmul_bfp_workspace_bytes.argtypes = [u32, u32, u32, u32, i32]
        L.ttmi_matmul_bfp.restype = i32
        L.ttmi_matmul_bfp.argtypes = [vp, i32, vp, i32, u32, u32, u32, u32, u32, vp, i32, vp, i32, i32, vp, sz, vp]
        L.ttmi_matmul_bfp_plan.restype = None
        L.ttmi_matmul_bfp_plan.argtypes = [u32, u32, u32, u32, i32, i32, i32, ctypes.POINTER(u32)]
        L.ttmi_matmul_bfp_ab_supported.restype = i32
        L.ttmi_matmul_bfp_ab_supported.argtypes = [u32, u32, u32, u32, i32, i32]
        L.ttmi_matmul_bfp_ab.restype = i32
        L.ttmi_matmul_bfp_ab.argtypes = [vp, i32, vp, i32, u32, u32, u32, u32, u32, vp, i32, vp, i32, i32, vp, sz, vp]
        L.ttmi_copy_window.restype = i32
        L.ttmi_copy_window.argtypes = [i32, vp, ctypes.POINTER(u32), vp, ctypes.POINTER(u32), ctypes.POINTER(ctypes.c_int32), ctypes.c_float, vp]
        L.ttmi_unpad_tiles.restype = i32
        L.ttmi_unpad_tiles.argtypes = [i32, vp, ctypes.POINTER(u32), vp, ctypes.POINTER(u32), ctypes.POINTER(u32), vp]
        L.ttmi_matmul_bfp_gated_workspace_bytes.restype = ctypes.c_size_t
        L.ttmi_matmul_bfp_gated_workspace_bytes.argtypes = [u32, u32, u32, u32, i32]
        L.ttmi_matmul_bfp_gated.restype = i32
        L.ttmi_matmul_bfp_gated.argtypes = [vp, i32, vp, vp, i32, u32, u32, u32, u32, u32, vp, i32, vp, i32, i32, vp, ctypes.c_size_t, vp]
        L.ttmi_matmul_bf16_workspace_bytes.restype = ctypes.c_size_t
        L.ttmi_matmul_bf16_workspace_bytes.argtypes = [u32, u32, u32]
        L.ttmi_matmul_bf16.restype = i32
        L.ttmi_matmul_bf16.argtypes = [vp, i32, vp, u32, u32, u32, u32, u32, vp, i32, vp, i32, i32, vp, ctypes.c_size_t, vp]
        L.ttmi_matmul_bfp_static.restype = i32
        L.ttmi_matmul_bfp_static.argtypes = [vp, i32, vp, i32, u32, u32, u32, u32, u32, vp, i32, vp, i32, i32, vp]
        L.ttmi_typecast_tiles.restype = i32
        L.ttmi_typecast_tiles.argtypes = [vp, i32, vp, i32, sz, vp]
        L.ttmi_device_status.restype = i32
        L.ttmi_device_status.argtypes = []
        L.ttmi_release_scratch.restype = i32
        L.ttmi_release_scratch.argtypes = [ctypes.POINTER(ctypes.c_size_t)]
        L.ttmi_eltwise_bf16.restype = i32
        L.ttmi_eltwise_bf16.argtypes = [i32, vp, vp, ctypes.c_float, vp, sz, vp]
        _loaded[path] = L
    return _loaded[path]


def check(status: int) -> None:
    if status != 0:
        raise RuntimeError(lib().ttmi_last_error().decode())


def _stream():
    import torch

    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(t):
    if not t.is_cuda:
        raise RuntimeError("ttmi kernels need device tensors (no CPU fallback)")
    return ctypes.c_void_p(t.data_ptr())


def _torch_dtype_code(t):
    import torch

    if t.dtype == torch.float32:
        return FLOAT32
    if t.dtype == torch.bfloat16:
        return BFLOAT16
    raise RuntimeError(f"unsupported source dtype {t.dtype}")


def padded(x: int) -> int:
    return (x + 31) // 32 * 32


# ---- torch-pointer helpers (device tensors in, device tensors out) -------------------------------------

def pack_chunks(fmt: int, src, row_major_input: bool):
    """src: cuda fp32, numel a multiple of 1024 -> cuda int32 words (mirrors pack_fp32_vec_as_bfp{8,4}_tiles)."""
    import torch

    assert src.dtype == torch.float32 and src.is_contiguous() and src.numel() % 1024 == 0
    n_tiles = src.numel() // 1024
    out = torch.empty(n_tiles * TILE_BYTES[fmt] // 4, dtype=torch.int32, device=src.device)
    check(lib().ttmi_pack_fp32_vec_as_bfp_tiles(fmt, _dev(src), n_tiles, int(row_major_input), _dev(out), _stream()))
    return out


def unpack_chunks(fmt: int, words, row_major_output: bool):
    import torch

    assert words.dtype == torch.int32 and words.is_contiguous()
    n_tiles = words.numel() * 4 // TILE_BYTES[fmt]
    out = torch.empty(n_tiles * 1024, dtype=torch.float32, device=words.device)
    check(lib().ttmi_unpack_bfp_tiles_into_float_vec(fmt, _dev(words), n_tiles, int(row_major_output), _dev(out), _stream()))
    return out


def _bhw(t):
    h, w = t.shape[-2], t.shape[-1]
    batch = 1
    for s in t.shape[:-2]:
        batch *= s
    return batch, h, w


def pack_tensor(fmt: int, src):
    """[..., H, W] cuda fp32/bf16 (dense) -> packed words of the padded, tilized tensor."""
    import torch

    src = src.contiguous()
    batch, h, w = _bhw(src)
    nbytes = lib().ttmi_tiled_size_bytes(fmt, batch, h, w)
    out = torch.empty(nbytes // 4, dtype=torch.int32, device=src.device)
    check(lib().ttmi_pack_rowmajor_as_bfp_tiles(fmt, _dev(src), _torch_dtype_code(src), batch, h, w, w, h * w, _dev(out), _stream()))
    return out


def unpack_tensor(fmt: int, words, shape, dtype=None):
    import torch

    dtype = dtype or torch.float32
    out = torch.empty(tuple(shape), dtype=dtype, device=words.device)
    batch, h, w = _bhw(out)
    check(lib().ttmi_unpack_bfp_tiles_as_rowmajor(fmt, _dev(words), batch, h, w, _dev(out), _torch_dtype_code(out), _stream()))
    return out


def tilize(src):
    """[..., H, W] dense cuda tensor with 2- or 4-byte elements -> flat tile-order tensor of the padded shape."""
    import torch

    src = src.contiguous()
    batch, h, w = _bhw(src)
    out = torch.empty(batch * padded(h) * padded(w), dtype=src.dtype, device=src.device)
    check(lib().ttmi_tilize(_dev(src), src.element_size(), batch, h, w, _dev(out), _stream()))
    return out


def untilize(tiles, shape):
    import torch

    out = torch.empty(tuple(shape), dtype=tiles.dtype, device=tiles.device)
    batch, h, w = _bhw(out)
    assert tiles.numel() == batch * padded(h) * padded(w)
    check(lib().ttmi_untilize(_dev(tiles), tiles.element_size(), batch, h, w, _dev(out), _stream()))
    return out


def matmul_bfp(a, a_layout: int, b_words, b_fmt: int, batch: int, b_batch: int, m: int, k: int, n: int, *,
               bias=None, activation: int = ACT_NONE, c_layout: int = ROW_MAJOR, out_dtype=None, workspace=None, out_bfp: int | None = None):
    """a: cuda bf16 (dense [batch,m,k] or tile order); b_words: packed weights; returns C (dense or tile order).
    out_bfp = BFLOAT8_B | BFLOAT4_B (TILE layout only): C as packed words."""
    import torch

    out_dtype = out_dtype or torch.bfloat16
    mp = padded(m) if c_layout == TILE else m
    if out_bfp is not None:
        c = torch.empty(batch * (mp // 32) * (n // 32) * TILE_BYTES[out_bfp] // 4, dtype=torch.int32, device=a.device)
    else:
        c = torch.empty(batch * mp * n, dtype=out_dtype, device=a.device)
    ws_ptr, ws_bytes = None, 0
    if workspace is not None:
        ws_ptr, ws_bytes = _dev(workspace), workspace.numel() * workspace.element_size()
    check(lib().ttmi_matmul_bfp(
        _dev(a), a_layout, _dev(b_words), b_fmt, batch, b_batch, m, k, n,
        _dev(bias) if bias is not None else None, activation, _dev(c), c_layout, out_bfp if out_bfp is not None else _torch_dtype_code(c),
        ws_ptr, ws_bytes, _stream()))
    if c_layout == ROW_MAJOR:
        return c.view(batch, m, n)
    return c


def matmul_bfp_ab(a_words, a_fmt: int, b_words, b_fmt: int, batch: int, b_batch: int, m: int, k: int, n: int, *,
                  bias=None, activation: int = ACT_NONE, c_layout: int = ROW_MAJOR, out_dtype=None, workspace=None, out_bfp: int | None = None):
    """Block-float activations (ttmi_matmul_bfp_ab): a_words = packed tiles of A; the rest as for matmul_bfp."""
    import torch

    out_dtype = out_dtype or torch.bfloat16
    if out_bfp is not None:
        c = torch.empty(batch * (m // 32) * (n // 32) * TILE_BYTES[out_bfp] // 4, dtype=torch.int32, device=a_words.device)
    else:
        c = torch.empty(batch * m * n, dtype=out_dtype, device=a_words.device)
    ws_ptr, ws_bytes = None, 0
    if workspace is not None:
        ws_ptr, ws_bytes = _dev(workspace), workspace.numel() * workspace.element_size()
    check(lib().ttmi_matmul_bfp_ab(
        _dev(a_words), a_fmt, _dev(b_words), b_fmt, batch, b_batch, m, k, n,
        _dev(bias) if bias is not None else None, activation, _dev(c), c_layout, out_bfp if out_bfp is not None else _torch_dtype_code(c),
        ws_ptr, ws_bytes, _stream()))
    return c.view(batch, m, n) if c_layout == ROW_MAJOR else c


def matmul_bf16(a, a_layout: int, b_tiles, batch: int, b_batch: int, m: int, k: int, n: int, *, bias=None, activation: int = ACT_NONE,
                c_layout: int = ROW_MAJOR, out_dtype=None, workspace=None):
    """bf16 x bf16 (ttmi_matmul_bf16): b_tiles = bf16 weights in TILE layout; the rest as for matmul_bfp."""
    import torch

    out_dtype = out_dtype or torch.bfloat16
    mp = padded(m) if c_layout == TILE else m
    c = torch.empty(batch * mp * n, dtype=out_dtype, device=a.device)
    ws_ptr, ws_bytes = None, 0
    if workspace is not None:
        ws_ptr, ws_bytes = _dev(workspace), workspace.numel() * workspace.element_size()
    check(lib().ttmi_matmul_bf16(_dev(a), a_layout, _dev(b_tiles), batch, b_batch, m, k, n, _dev(bias) if bias is not None else None, activation,
                                 _dev(c), c_layout, _torch_dtype_code(c), ws_ptr, ws_bytes, _stream()))
    return c.view(batch, m, n) if c_layout == ROW_MAJOR else c


def matmul_bfp_gated(a, a_layout: int, gate_words, up_words, b_fmt: int, batch: int, b_batch: int, m: int, k: int, n: int, *,
                     bias=None, activation: int = ACT_SILU, c_layout: int = ROW_MAJOR, out_dtype=None, workspace=None, out_bfp=None):
    """act(a . gate + bias) * (a . up) in one launch (ttmi_matmul_bfp_gated); arguments as for matmul_bfp."""
    import torch

    out_dtype = out_dtype or torch.bfloat16
    mp = padded(m) if c_layout == TILE else m
    if out_bfp is not None:
        c = torch.empty(lib().ttmi_tiled_size_bytes(out_bfp, batch, m, n) // 4, dtype=torch.int32, device=a.device)
    else:
        c = torch.empty(batch * mp * n, dtype=out_dtype, device=a.device)
    ws_ptr, ws_bytes = None, 0
    if workspace is not None:
        ws_ptr, ws_bytes = _dev(workspace), workspace.numel() * workspace.element_size()
    check(lib().ttmi_matmul_bfp_gated(
        _dev(a), a_layout, _dev(gate_words), _dev(up_words), b_fmt, batch, b_batch, m, k, n,
        _dev(bias) if bias is not None else None, activation, _dev(c), c_layout, out_bfp if out_bfp is not None else _torch_dtype_code(c),
        ws_ptr, ws_bytes, _stream()))
    if c_layout == ROW_MAJOR:
        return c.view(batch, m, n)
    return c


def eltwise(op: int, a, b=None, scalar: float = 0.0):
    """op(a, b) (or op(a, scalar), or a unary op of a) on cuda bf16 tensors with equal element counts; returns a tensor like a."""
    import torch

    if a.dtype != torch.bfloat16 or (b is not None and b.dtype != torch.bfloat16):
        raise RuntimeError("eltwise: operands must be bfloat16")
    if b is not None and b.numel() != a.numel():
        raise RuntimeError("eltwise: operands must have the same number of elements")
    a = a.contiguous()
    b = b.contiguous() if b is not None else None
    out = torch.empty_like(a)
    check(lib().ttmi_eltwise_bf16(op, _dev(a), _dev(b) if b is not None else None, float(scalar), _dev(out), a.numel(), _stream()))
    return out


def copy_window(dtype: int, src, src_shape, dst_shape, offset, fill: float = 0.0):
    """Tensor::pad / unpad on a cuda buffer: dst[i] = src[i - offset] inside src, `fill` elsewhere (4-D shapes).
    Dense dtypes return a tensor of dst_shape; block-float dtypes take and return flat packed words."""
    import torch

    src_shape = tuple(int(x) for x in src_shape)
    dst_shape = tuple(int(x) for x in dst_shape)
    volume = 1
    for x in dst_shape:
        volume *= x
    if dtype in (BFLOAT8_B, BFLOAT4_B):
        out = torch.empty(volume // 1024 * (TILE_BYTES[dtype] // 4), dtype=src.dtype, device=src.device)
    else:
        out = torch.empty(dst_shape, dtype=src.dtype, device=src.device)
    check(lib().ttmi_copy_window(dtype, _dev(src.contiguous()), (ctypes.c_uint32 * 4)(*src_shape), _dev(out), (ctypes.c_uint32 * 4)(*dst_shape),
                                 (ctypes.c_int32 * 4)(*[int(x) for x in offset]), float(fill), _stream()))
    return out


def unpad_tiles(dtype: int, tiles, src_tiles, start_tile, dst_tiles):
    """Whole tiles [start_tile, start_tile + dst_tiles) of a TILE-layout cuda buffer with tile grid src_tiles (4-D)."""
    import torch

    count = 1
    for x in dst_tiles:
        count *= int(x)
    per_tile = TILE_BYTES[dtype] // tiles.element_size()
    out = torch.empty(count * per_tile, dtype=tiles.dtype, device=tiles.device)
    u4 = ctypes.c_uint32 * 4
    check(lib().ttmi_unpad_tiles(dtype, _dev(tiles.contiguous()), u4(*[int(x) for x in src_tiles]), _dev(out), u4(*[int(x) for x in start_tile]),
                                 u4(*[int(x) for x in dst_tiles]), _stream()))
    return out


def release_scratch() -> int:
    """Frees the library's own device buffers on the current device (after the device has gone idle); returns the bytes freed."""
    freed = ctypes.c_size_t(0)
    check(lib().ttmi_release_scratch(ctypes.byref(freed)))
    return int(freed.value)


def device_status() -> None:
    """Raises what a kernel on the current device has reported since the last query (a wait that gave up)."""
    check(lib().ttmi_device_status())


_TORCH_OF = {}


def typecast_tiles(src, src_dtype: int, dst_dtype: int):
    """A flat cuda buffer in tile order from one data type to another (block-float <-> bf16 / fp32, bf16 <-> fp32), one kernel."""
    import torch

    if not _TORCH_OF:
        _TORCH_OF.update({BFLOAT16: torch.bfloat16, FLOAT32: torch.float32, BFLOAT8_B: torch.int32, BFLOAT4_B: torch.int32})
    src = src.contiguous().reshape(-1)
    nbytes = src.numel() * src.element_size()
    if nbytes % TILE_BYTES[src_dtype]:
        raise RuntimeError("typecast: the buffer does not hold whole tiles")
    n_tiles = nbytes // TILE_BYTES[src_dtype]
    out = torch.empty(n_tiles * TILE_BYTES[dst_dtype] // torch.empty(0, dtype=_TORCH_OF[dst_dtype]).element_size(), dtype=_TORCH_OF[dst_dtype],
                      device=src.device)
    check(lib().ttmi_typecast_tiles(_dev(src), src_dtype, _dev(out), dst_dtype, n_tiles, _stream()))
    return out
