"""numpy front end of the CPU oracle (``bfp_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; the product path never touches it.

Each wrapper hands numpy buffers to the C restatement of the reference host codecs
(``tt_metal/common/bfloat8.hpp``, ``bfloat4.hpp``, ``blockfloat_common.hpp``,
``test_tiles.hpp``, ``tilize_untilize.hpp``); see the C file for the line-level citations.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

BFP8_B = 3  # tt_eager/tensor/types.hpp:24-34
BFP4_B = 4
TILE_WORDS = {BFP8_B: 272, BFP4_B: 144}
TILE_BYTES = {BFP8_B: 1088, BFP4_B: 576}

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libbfp_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (seconds); returns the library path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True, capture_output=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, u32, i32, sz = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_int, ctypes.c_size_t
        L.oracle_tile_size_bytes.restype = u32
        L.oracle_tile_size_bytes.argtypes = [i32]
        L.oracle_get_max_exp.restype = u32
        L.oracle_get_max_exp.argtypes = [vp]
        L.oracle_convert_u32_to_bfp.restype = u32
        L.oracle_convert_u32_to_bfp.argtypes = [u32, u32, i32]
        L.oracle_bfp_code_to_u32.restype = u32
        L.oracle_bfp_code_to_u32.argtypes = [u32, u32, i32]
        L.oracle_pack_fp32_vec_as_bfp_tiles.restype = None
        L.oracle_pack_fp32_vec_as_bfp_tiles.argtypes = [i32, vp, sz, i32, vp]
        L.oracle_unpack_bfp_tiles_into_float_vec.restype = None
        L.oracle_unpack_bfp_tiles_into_float_vec.argtypes = [i32, vp, sz, i32, vp]
        for name in ("oracle_tilize_nchw_4faces", "oracle_untilize_nchw_4faces"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, u32, u32, u32, u32, u32, vp]
        for name in ("oracle_tilize_bf16_blocks", "oracle_untilize_bf16_blocks"):
            getattr(L, name).restype = i32
            getattr(L, name).argtypes = [vp, sz, u32, u32, vp]
        for name in ("oracle_from_torch_bfp_tiles", "oracle_to_torch_bfp_tiles"):
            getattr(L, name).restype = i32
            getattr(L, name).argtypes = [i32, vp, u32, u32, u32, vp]
        L.oracle_pad_rowmajor.restype = i32
        L.oracle_pad_rowmajor.argtypes = [vp, u32, vp, vp, vp, vp, vp]
        L.oracle_unpad_rowmajor.restype = i32
        L.oracle_unpad_rowmajor.argtypes = [vp, u32, vp, vp, vp, vp]
        L.oracle_pad_bfp.restype = i32
        L.oracle_pad_bfp.argtypes = [i32, vp, vp, vp, vp, ctypes.c_float, vp]
        L.oracle_unpad_bfp.restype = i32
        L.oracle_unpad_bfp.argtypes = [i32, vp, vp, vp, vp, vp]
        L.oracle_bf16_truncate.restype = ctypes.c_uint16
        L.oracle_bf16_truncate.argtypes = [ctypes.c_float]
        L.oracle_gold_bmm.restype = None
        L.oracle_gold_bmm.argtypes = [vp, vp, u32, u32, u32, u32, vp, vp]
        _lib = L
    return _lib


def _ptr(a: np.ndarray) -> ctypes.c_void_p:
    return ctypes.c_void_p(a.ctypes.data)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def convert_u32_to_bfp(bits: int, shared_exp: int, fmt: int) -> int:
    return int(lib().oracle_convert_u32_to_bfp(bits & 0xFFFFFFFF, shared_exp, fmt))


def bfp_code_to_u32(code: int, shared_exp: int, fmt: int) -> int:
    return int(lib().oracle_bfp_code_to_u32(code, shared_exp, fmt))


def get_max_exp(row16_bits) -> int:
    row = _c(row16_bits, np.uint32)
    assert row.size == 16
    return int(lib().oracle_get_max_exp(_ptr(row)))


def pack_fp32_vec_as_bfp_tiles(fmt: int, values, row_major_input: bool) -> np.ndarray:
    """1024-element chunks of fp32 -> packed tile words (uint32)."""
    src = _c(values, np.float32).reshape(-1)
    assert src.size % 1024 == 0
    n_tiles = src.size // 1024
    out = np.empty(n_tiles * TILE_WORDS[fmt], dtype=np.uint32)
    lib().oracle_pack_fp32_vec_as_bfp_tiles(fmt, _ptr(src), n_tiles, int(row_major_input), _ptr(out))
    return out


def unpack_bfp_tiles_into_float_vec(fmt: int, words, row_major_output: bool) -> np.ndarray:
    w = _c(words, np.uint32).reshape(-1)
    assert w.size % TILE_WORDS[fmt] == 0
    n_tiles = w.size // TILE_WORDS[fmt]
    out = np.empty(n_tiles * 1024, dtype=np.float32)
    lib().oracle_unpack_bfp_tiles_into_float_vec(fmt, _ptr(w), n_tiles, int(row_major_output), _ptr(out))
    return out


def tilize_nchw_4faces(x: np.ndarray) -> np.ndarray:
    """[N,C,H,W] row-major (any 2- or 4-byte dtype) -> zero-padded 4-face tile order, flat."""
    x = np.ascontiguousarray(x)
    n, c, h, w = x.shape
    hp, wp = -(-h // 32) * 32, -(-w // 32) * 32
    out = np.empty(n * c * hp * wp, dtype=x.dtype)
    lib().oracle_tilize_nchw_4faces(_ptr(x), n, c, h, w, x.dtype.itemsize, _ptr(out))
    return out


def untilize_nchw_4faces(flat: np.ndarray, shape) -> np.ndarray:
    n, c, h, w = shape
    assert h % 32 == 0 and w % 32 == 0
    flat = np.ascontiguousarray(flat).reshape(-1)
    assert flat.size == n * c * h * w
    out = np.empty((n, c, h, w), dtype=flat.dtype)
    lib().oracle_untilize_nchw_4faces(_ptr(flat), n, c, h, w, flat.dtype.itemsize, _ptr(out))
    return out


def tilize_bf16_blocks(values_u16, m: int, n: int) -> np.ndarray:
    src = _c(values_u16, np.uint16).reshape(-1)
    out = np.empty_like(src)
    if lib().oracle_tilize_bf16_blocks(_ptr(src), src.size, m, n, _ptr(out)) != 0:
        raise RuntimeError("tilize: size, m and n must be non-zero, size divisible by m*n, m and n divisible by 32")
    return out


def untilize_bf16_blocks(values_u16, m: int, n: int) -> np.ndarray:
    src = _c(values_u16, np.uint16).reshape(-1)
    out = np.empty_like(src)
    if lib().oracle_untilize_bf16_blocks(_ptr(src), src.size, m, n, _ptr(out)) != 0:
        raise RuntimeError("untilize: size, m and n must be non-zero, size divisible by m*n, m and n divisible by 32")
    return out


def from_torch_bfp_tiles(fmt: int, x: np.ndarray) -> np.ndarray:
    """[..., H, W] fp32 -> packed words of the zero-padded, tilized tensor (the reference's full host sequence)."""
    x = _c(x, np.float32)
    h, w = x.shape[-2:]
    batch = int(np.prod(x.shape[:-2], dtype=np.int64)) if x.ndim > 2 else 1
    hp, wp = -(-h // 32) * 32, -(-w // 32) * 32
    out = np.empty(batch * (hp // 32) * (wp // 32) * TILE_WORDS[fmt], dtype=np.uint32)
    if lib().oracle_from_torch_bfp_tiles(fmt, _ptr(x), batch, h, w, _ptr(out)) != 0:
        raise MemoryError
    return out


def to_torch_bfp_tiles(fmt: int, words, shape) -> np.ndarray:
    """packed words of a padded tilized tensor -> fp32 array of logical ``shape`` (full host sequence)."""
    shape = tuple(int(s) for s in shape)
    h, w = shape[-2:]
    batch = int(np.prod(shape[:-2], dtype=np.int64)) if len(shape) > 2 else 1
    wds = _c(words, np.uint32).reshape(-1)
    hp, wp = -(-h // 32) * 32, -(-w // 32) * 32
    assert wds.size == batch * (hp // 32) * (wp // 32) * TILE_WORDS[fmt]
    out = np.empty(shape, dtype=np.float32)
    if lib().oracle_to_torch_bfp_tiles(fmt, _ptr(wds), batch, h, w, _ptr(out)) != 0:
        raise MemoryError
    return out


def _shape4(shape) -> np.ndarray:
    shape = tuple(int(x) for x in shape)
    assert len(shape) == 4, "pad / unpad work on 4-D shapes (tt_eager/tensor/tensor_impl.hpp:508-660)"
    return np.array(shape, dtype=np.uint32)


def pad_rowmajor(x: np.ndarray, output_shape, input_start, pad_value) -> np.ndarray:
    """Tensor::pad of a 4-D row-major array with 2- or 4-byte elements; pad_value is converted by numpy to x's dtype."""
    x = np.ascontiguousarray(x)
    out = np.empty(tuple(int(v) for v in output_shape), dtype=x.dtype)
    pad = np.array([pad_value], dtype=x.dtype)
    in_s, out_s, at = _shape4(x.shape), _shape4(output_shape), _shape4(input_start)      # kept alive across the call
    if lib().oracle_pad_rowmajor(_ptr(x), x.dtype.itemsize, _ptr(in_s), _ptr(out_s), _ptr(at), _ptr(pad), _ptr(out)) != 0:
        raise RuntimeError("pad: the input does not fit into the output at that position")
    return out


def unpad_rowmajor(x: np.ndarray, start, end) -> np.ndarray:
    """Tensor::unpad: elements start..end (inclusive) of a 4-D row-major array."""
    x = np.ascontiguousarray(x)
    out = np.empty(tuple(int(e) - int(s) + 1 for s, e in zip(start, end)), dtype=x.dtype)
    in_s, lo, hi = _shape4(x.shape), _shape4(start), _shape4(end)
    if lib().oracle_unpad_rowmajor(_ptr(x), x.dtype.itemsize, _ptr(in_s), _ptr(lo), _ptr(hi), _ptr(out)) != 0:
        raise RuntimeError("unpad: start / end outside the tensor")
    return out


def pad_bfp(fmt: int, words, input_shape, output_shape, input_start, pad_value: float) -> np.ndarray:
    """pad_bfloat8_b / pad_bfloat4_b: words of a block-float tensor declared ROW_MAJOR (sequential 1024-chunks)."""
    w = _c(words, np.uint32).reshape(-1)
    out_vol = int(np.prod(_shape4(output_shape), dtype=np.int64))
    out = np.empty(out_vol // 1024 * TILE_WORDS[fmt], dtype=np.uint32)
    in_s, out_s, at = _shape4(input_shape), _shape4(output_shape), _shape4(input_start)
    if lib().oracle_pad_bfp(fmt, _ptr(w), _ptr(in_s), _ptr(out_s), _ptr(at), float(pad_value), _ptr(out)) != 0:
        raise RuntimeError("pad: shapes must hold whole 1024-element chunks and the input must fit")
    return out


def unpad_bfp(fmt: int, words, input_shape, start, end) -> np.ndarray:
    w = _c(words, np.uint32).reshape(-1)
    out_vol = int(np.prod([int(e) - int(s) + 1 for s, e in zip(start, end)], dtype=np.int64))
    out = np.empty(max(out_vol // 1024, 0) * TILE_WORDS[fmt], dtype=np.uint32)
    in_s, lo, hi = _shape4(input_shape), _shape4(start), _shape4(end)
    if lib().oracle_unpad_bfp(fmt, _ptr(w), _ptr(in_s), _ptr(lo), _ptr(hi), _ptr(out)) != 0:
        raise RuntimeError("unpad: shapes must hold whole 1024-element chunks and start / end must lie inside the tensor")
    return out


def bf16_truncate(x) -> np.ndarray:
    """fp32 -> bf16 bit patterns by dropping the low 16 bits (bfloat16.hpp:28-38)."""
    return (_c(x, np.float32).view(np.uint32) >> 16).astype(np.uint16)


def bf16_to_f32(bits_u16) -> np.ndarray:
    return (_c(bits_u16, np.uint16).astype(np.uint32) << 16).view(np.float32)


def gold_bmm(a_bf16_bits, b_bf16_bits, nb: int, m: int, k: int, n: int):
    """gold_bmm: returns (fp32 result, bf16-truncated bits), both [nb, m, n]."""
    a = _c(a_bf16_bits, np.uint16).reshape(nb, m, k)
    b = _c(b_bf16_bits, np.uint16).reshape(nb, k, n)
    f = np.empty((nb, m, n), dtype=np.float32)
    h = np.empty((nb, m, n), dtype=np.uint16)
    lib().oracle_gold_bmm(_ptr(a), _ptr(b), nb, m, k, n, _ptr(f), _ptr(h))
    return f, h


def matmul_reference(a_f32: np.ndarray, w_unpacked_f32: np.ndarray) -> np.ndarray:
    """fp32 CPU matmul on unpacked weights: the parity target for the block-float GEMM.
    Accumulates in float64 and rounds once to fp32, so it is a tight centre for the error bound."""
    return np.matmul(a_f32.astype(np.float64), w_unpacked_f32.astype(np.float64)).astype(np.float32)
