"""The tensor-file format of ttnn.dump_tensor / load_tensor (tt_eager/tensor/serialization.cpp:86-141) on the CPU.

The header is the raw memory of the reference's `Shape` object.  What pins its layout here is an independent statement of
that class's members (tt_eager/tensor/types.hpp:46-63 Padding, :118-121 Shape) as ctypes structures, which follow the
platform's C ABI exactly as the reference's compiler does: offsets and the size 184 come from the member list, not from the
byte string tt_lib/tensor.py writes.
"""
import ctypes
import struct

import pytest
import torch

import tt_lib as ttl
import ttnn


class PadDimension(ctypes.Structure):       # types.hpp:49-55
    _fields_ = [("front", ctypes.c_size_t), ("back", ctypes.c_size_t)]


class Padding(ctypes.Structure):            # types.hpp:57-59: rank_, pad_dimensions_, pad_value_ (enum class = int)
    _fields_ = [("rank_", ctypes.c_size_t), ("pad_dimensions_", PadDimension * 8), ("pad_value_", ctypes.c_int)]


class Shape(ctypes.Structure):              # types.hpp:119-121: rank_, dimensions_, padding_
    _fields_ = [("rank_", ctypes.c_size_t), ("dimensions_", ctypes.c_uint32 * 8), ("padding_", Padding)]


def test_header_layout_follows_the_member_declarations():
    assert ctypes.sizeof(Shape) == 184
    assert (Shape.rank_.offset, Shape.dimensions_.offset, Shape.padding_.offset) == (0, 8, 40)
    assert (Padding.rank_.offset, Padding.pad_dimensions_.offset, Padding.pad_value_.offset) == (0, 8, 136)


def test_dumped_file_parses_as_the_reference_struct(tmp_path):
    x = torch.arange(2 * 5 * 3, dtype=torch.float32).reshape(2, 5, 3)
    t = ttl.tensor.Tensor(x)
    name = tmp_path / "t.bin"
    ttnn.dump_tensor(name, t)
    raw = name.read_bytes()
    shape = Shape.from_buffer_copy(raw[:184])
    assert shape.rank_ == 3 and list(shape.dimensions_) == [2, 5, 3, 0, 0, 0, 0, 0]
    assert shape.padding_.rank_ == 3 and shape.padding_.pad_value_ == 0
    assert all(p.front == 0 and p.back == 0 for p in shape.padding_.pad_dimensions_)
    dtype, layout, count = struct.unpack("<iiQ", raw[184:200])
    assert (dtype, layout, count) == (int(ttnn.float32), int(ttnn.ROW_MAJOR_LAYOUT), 30)
    assert raw[200:] == x.numpy().tobytes() and len(raw) == 200 + 120


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.int32, torch.int16])
def test_dump_and_load_round_trip_on_the_host(tmp_path, dtype):
    """tests/ttnn/unit_tests/test_dump_and_load.py:14-25 for every host dtype."""
    torch.manual_seed(3)
    x = (torch.rand((64, 48)) * 100).to(dtype)
    t = ttnn.from_torch(x)
    ttnn.dump_tensor(tmp_path / "tensor.bin", t)
    back = ttnn.load_tensor(tmp_path / "tensor.bin")
    assert back.dtype == t.dtype and back.layout == t.layout and back.shape == t.shape
    assert not ttnn.is_tensor_storage_on_device(back)
    assert torch.equal(ttnn.to_torch(back), x)


def test_padding_is_kept(tmp_path):
    """A tensor whose padded shape differs from its logical one: the header carries both (dims = padded, pad back = the difference)."""
    buf = torch.zeros(32 * 32, dtype=torch.bfloat16)
    t = ttl.tensor.Tensor(None, _raw=(buf, (7, 3), (32, 32), ttl.tensor.DataType.BFLOAT16, ttl.tensor.Layout.TILE, None))
    ttnn.dump_tensor(tmp_path / "p.bin", t)
    shape = Shape.from_buffer_copy((tmp_path / "p.bin").read_bytes()[:184])
    assert list(shape.dimensions_)[:2] == [32, 32]
    assert [(p.front, p.back) for p in shape.padding_.pad_dimensions_][:2] == [(0, 25), (0, 29)]
    back = ttnn.load_tensor(tmp_path / "p.bin")
    assert tuple(back.shape) == (7, 3) and tuple(back.shape.with_tile_padding()) == (32, 32) and back.layout == ttnn.TILE_LAYOUT


def test_errors(tmp_path):
    with pytest.raises(RuntimeError, match="does not exist"):
        ttnn.load_tensor(tmp_path / "missing.bin")
    with pytest.raises(RuntimeError, match="is not a file"):
        ttnn.load_tensor(tmp_path)
    (tmp_path / "short.bin").write_bytes(b"\0" * 50)
    with pytest.raises(RuntimeError, match="too short"):
        ttnn.load_tensor(tmp_path / "short.bin")
    ttnn.dump_tensor(tmp_path / "ok.bin", ttnn.from_torch(torch.ones(4, 4)))
    data = (tmp_path / "ok.bin").read_bytes()
    (tmp_path / "cut.bin").write_bytes(data[:-8])
    with pytest.raises(RuntimeError, match="ends inside"):
        ttnn.load_tensor(tmp_path / "cut.bin")
    # a header whose element count is not what its shape says (a stale or truncated cache file): refused before any kernel
    # could index the buffer by the shape
    (tmp_path / "count.bin").write_bytes(data[:192] + struct.pack("<Q", 8) + data[200:232])
    with pytest.raises(RuntimeError, match="the header counts 8 elements"):
        ttnn.load_tensor(tmp_path / "count.bin")
    header = bytearray(data[:200])
    header[48 + 8:48 + 16] = struct.pack("<Q", 9)            # Padding::pad_dimensions_[0].back = 9 on a dimension of 4
    (tmp_path / "pad.bin").write_bytes(bytes(header) + data[200:])
    with pytest.raises(RuntimeError, match="exceeds the dimension"):
        ttnn.load_tensor(tmp_path / "pad.bin")
