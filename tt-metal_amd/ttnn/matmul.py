"""ttnn.matmul / ttnn.linear (ttnn/ttnn/operations/matmul.py:295-416,441-516; ttnn/cpp/ttnn/operations/matmul.hpp:44-214)."""
from __future__ import annotations

from typing import Optional

import ttnn
from tt_lib.tensor import DataType, Layout, Tensor, _matmul
from ttmi import capi

_ACT = {None: capi.ACT_NONE, "relu": capi.ACT_RELU, "gelu": capi.ACT_GELU, "silu": capi.ACT_SILU}


def _validate(operation_name, t: Tensor, name: str):
    # validation.hpp:17-74 through matmul.hpp:39-42: rank 2-4; bf16 | bfp8_b | bfp4_b; TILE; on device
    if not isinstance(t, Tensor):
        raise RuntimeError(f"{operation_name}: {name} must be a ttnn.Tensor")
    if len(t._shape) not in (2, 3, 4):
        raise RuntimeError(f"{operation_name}: Tensor must be of rank (2, 3, 4), but got {len(t._shape)}")
    if t.dtype not in (DataType.BFLOAT16, DataType.BFLOAT8_B, DataType.BFLOAT4_B):
        raise RuntimeError(f"{operation_name}: Tensor must be of type bfloat16, bfloat8_b or bfloat4_b, but got {t.dtype.name}")
    if t.layout != Layout.TILE:
        raise RuntimeError(f"{operation_name}: Tensor must be of layout TILE, but got {t.layout.name}")
    if not ttnn.is_tensor_storage_on_device(t):
        raise RuntimeError(f"{operation_name}: Tensor must be on device!")


def _run(operation_name, a, b, bias, activation, dtype):
    _validate(operation_name, a, "input_tensor_a")
    _validate(operation_name, b, "input_tensor_b")
    if activation not in _ACT:
        raise RuntimeError(f"{activation} is not supported as activation function. Use one of these instead: {[k for k in _ACT if k]}")
    if a._padded[-1] != b._padded[-2] or a._shape[-1] != b._shape[-2]:
        raise RuntimeError("The width of the first tensor must be equal to the height of the second tensor")  # matmul.hpp:60-62
    batch_b = 1
    for s in b._padded[:-2]:
        batch_b *= s
    if batch_b != 1 and activation is not None:
        raise RuntimeError("Cannot use activation with batched input b")  # matmul.py:215-216
    if bias is not None:
        _validate(operation_name, bias, "bias")
    return _matmul(a, b, bcast_batch=batch_b == 1, bias=bias, activation=_ACT[activation], output_dtype=dtype, op=operation_name)


def matmul(input_tensor_a: Tensor, input_tensor_b: Tensor, *, memory_config=None, dtype: Optional[DataType] = None,
           core_grid=None, program_config=None, use_1d_systolic_array: Optional[bool] = None, compute_kernel_config=None) -> Tensor:
    """C = A @ B, B's batch dimensions either all 1 (broadcast) or equal to A's.  Output: bfloat16, TILE layout, on device."""
    return _run("ttnn.matmul", input_tensor_a, input_tensor_b, None, None, dtype)


def linear(input_tensor_a: Tensor, input_tensor_b: Tensor, *, bias: Optional[Tensor] = None, memory_config=None,
           dtype: Optional[DataType] = None, core_grid=None, program_config=None, activation: Optional[str] = None,
           use_1d_systolic_array: Optional[bool] = None, compute_kernel_config=None) -> Tensor:
    """act(A @ B + bias): bias row-broadcast, activation in {None, "relu", "gelu", "silu"}, fused into the GEMM epilogue."""
    return _run("ttnn.linear", input_tensor_a, input_tensor_b, bias, activation, dtype)
