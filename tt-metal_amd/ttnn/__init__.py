"""TT-NN surface for the block-float hot path on MI355X.

Mirrors ttnn/ttnn/types.py:11-48, ttnn/ttnn/operations/core.py (from_torch, to_torch, to_layout, to_device,
from_device, reshape) and ttnn/ttnn/operations/matmul.py (matmul, linear) of tt-metal, same names, keyword
arguments and error conditions.  A signature shim: the Tensor object, the shape and padding rules, validation and
dispatch live in the C++ host layer of the pybind11 module ``_ttmi``; conversions and the GEMM run as HIP kernels behind
the C ABI.  Nothing computes on the CPU, and without the built library or without a GPU these functions raise RuntimeError.
Tensix-only knobs (core grids, program configs, math fidelity, memory configs) are accepted and ignored.
"""
from __future__ import annotations

from typing import Optional, Tuple, Union

import tt_lib as ttl

from tt_lib.tensor import DataType, Layout, StorageType, MemoryConfig, BufferType, TensorMemoryLayout, MathFidelity, Device, Tensor
from tt_lib.tensor import GrayskullComputeKernelConfig, WormholeComputeKernelConfig  # noqa: F401  (accepted by matmul / linear and ignored)
from ttmi import capi as _capi

# ---- ttnn/ttnn/types.py ----------------------------------------------------------------------------------
uint16 = DataType.UINT16
uint32 = DataType.UINT32
float32 = DataType.FLOAT32
bfloat16 = DataType.BFLOAT16
bfloat8_b = DataType.BFLOAT8_B
bfloat4_b = DataType.BFLOAT4_B

DRAM_MEMORY_CONFIG = MemoryConfig(TensorMemoryLayout.INTERLEAVED, BufferType.DRAM)
L1_MEMORY_CONFIG = MemoryConfig(TensorMemoryLayout.INTERLEAVED, BufferType.L1)

ROW_MAJOR_LAYOUT = Layout.ROW_MAJOR
TILE_LAYOUT = Layout.TILE
DEVICE_STORAGE_TYPE = StorageType.DEVICE
MULTI_DEVICE_STORAGE_TYPE = StorageType.MULTI_DEVICE
TILE_SIZE = 32


class Shape:
    """Logical shape plus the shape with tile padding (ttnn/cpp/pybind11/types.hpp; tests/ttnn/unit_tests/test_shape.py)."""

    def __init__(self, shape, full_shape=None):
        if isinstance(shape, Shape):
            full_shape = full_shape if full_shape is not None else shape._full
            shape = shape._value
        self._value = tuple(int(s) for s in shape)
        self._full = tuple(int(s) for s in (full_shape if full_shape is not None else shape))
        if len(self._value) != len(self._full):
            raise RuntimeError("Shape: rank of the shape and of the shape with tile padding differ")

    @property
    def rank(self):
        return len(self._value)

    def with_tile_padding(self) -> "Shape":
        return Shape(self._full, self._full)

    def __len__(self):
        return len(self._value)

    def __iter__(self):
        return iter(self._value)

    def __getitem__(self, i):
        if isinstance(i, slice):
            return Shape(self._value[i], self._full[i])
        return self._value[i]

    def __eq__(self, other):
        if isinstance(other, Shape):
            return self._value == other._value and self._full == other._full
        try:
            return self._value == tuple(other)
        except TypeError:
            return NotImplemented

    def __ne__(self, other):
        r = self.__eq__(other)
        return r if r is NotImplemented else not r

    def __hash__(self):
        return hash((self._value, self._full))

    def __repr__(self):
        if self._value == self._full:
            return f"ttnn.Shape({list(self._value)})"
        parts = [f"{v}[{f}]" if v != f else str(v) for v, f in zip(self._value, self._full)]
        return f"ttnn.Shape([{', '.join(parts)}])"


class CoreGrid:
    """Tensix core grid: accepted and ignored."""

    def __init__(self, y: int = 1, x: int = 1):
        self.y, self.x = y, x

    @property
    def num_cores(self):
        return self.x * self.y


# ---- devices (ttnn/ttnn/device.py) ------------------------------------------------------------------------
def open_device(device_id: int = 0, **_) -> Device:
    return Device(device_id)


def close_device(device: Device) -> None:
    synchronize_device(device)


def synchronize_device(device: Optional[Device] = None) -> None:
    import torch

    torch.cuda.synchronize()


def to_memory_config(tensor: Tensor, memory_config=None) -> Tensor:
    """ttnn/ttnn/operations/core.py:484-606 moves a tensor between DRAM, L1 and sharded layouts of a Tensix device.  One GPU has
    one memory, HBM, and every tensor is interleaved in it: an interleaved target is where the tensor already is; a sharded
    one has no meaning here and raises."""
    layout = getattr(memory_config, "memory_layout", None)
    if layout is not None and layout != TensorMemoryLayout.INTERLEAVED:
        raise RuntimeError("ttnn.to_memory_config: sharded memory configs describe Tensix L1 and are not supported on this device")
    return tensor


def is_tensor_storage_on_device(tensor: Tensor) -> bool:
    return tensor.storage_type() in (DEVICE_STORAGE_TYPE, MULTI_DEVICE_STORAGE_TYPE)


from .core import from_torch, to_torch, to_layout, to_device, from_device, reshape, deallocate, unsqueeze_to_4D, clone  # noqa: E402
from .matmul import matmul, linear, create_matmul_1d_systolic_array_program_config  # noqa: E402
from . import experimental  # noqa: E402
from .elementwise import mul, multiply, add, sub, subtract, gelu, relu, silu  # noqa: E402
from .files import load_tensor, dump_tensor, as_tensor, get_memory_config  # noqa: E402

Tensor.__matmul__ = lambda self, other: matmul(self, other)  # ttnn/ttnn/operations/matmul.py:519
