"""ttnn.mul / add / sub (ttnn/ttnn/operations/binary.py:200-424) and ttnn.gelu / relu / silu
(ttnn/ttnn/operations/unary.py), for tensors of equal shape or a tensor and a number: what the MLP blocks around the
block-float GEMMs use.  The broadcast forms (a [.., 1, W], [.., H, 1] or [.., 1, 1] second operand) are not built."""
from __future__ import annotations

from numbers import Number
from typing import Union

import ttnn
import tt_lib as ttl
from tt_lib.tensor import Tensor


def _binary(name, tensor_fn, unary_fn, input_tensor_a, input_tensor_b):
    if not isinstance(input_tensor_a, Tensor):
        raise TypeError("Expected first argument to be a ttnn.Tensor")                      # binary.py:352-353
    if not ttnn.is_tensor_storage_on_device(input_tensor_a):
        raise RuntimeError("input_tensor_a must be on device!")                             # binary.py:355-356
    if isinstance(input_tensor_b, Number):
        if unary_fn is None:
            raise RuntimeError(f"{name}: a number as second operand is not supported")
        return unary_fn(input_tensor_a, float(input_tensor_b))
    if not isinstance(input_tensor_b, Tensor):
        raise TypeError("Expected second argument to be a ttnn.Tensor or a scalar")          # binary.py:367-368
    if tuple(input_tensor_a.shape) != tuple(input_tensor_b.shape):
        raise RuntimeError(f"{name}: broadcasting {tuple(input_tensor_b.shape)} over {tuple(input_tensor_a.shape)} is not part of this build")
    return tensor_fn(input_tensor_a, input_tensor_b)


def mul(input_tensor_a: Tensor, input_tensor_b: Union[Tensor, Number], *, memory_config=None) -> Tensor:
    return _binary("ttnn.mul", ttl.tensor.mul, ttl.tensor.mul_unary, input_tensor_a, input_tensor_b)


def add(input_tensor_a: Tensor, input_tensor_b: Union[Tensor, Number], *, memory_config=None, alpha=1) -> Tensor:
    if alpha != 1:
        raise RuntimeError("ttnn.add: alpha other than 1 is not part of this build")
    return _binary("ttnn.add", ttl.tensor.add, ttl.tensor.add_unary, input_tensor_a, input_tensor_b)


def sub(input_tensor_a: Tensor, input_tensor_b: Union[Tensor, Number], *, memory_config=None, alpha=1) -> Tensor:
    if alpha != 1:
        raise RuntimeError("ttnn.sub: alpha other than 1 is not part of this build")
    return _binary("ttnn.sub", ttl.tensor.sub, None, input_tensor_a, input_tensor_b)


multiply = mul
subtract = sub


def _unary(name, fn, input_tensor):
    if not isinstance(input_tensor, Tensor):
        raise TypeError("Expected first argument to be a ttnn.Tensor")
    if not ttnn.is_tensor_storage_on_device(input_tensor):
        raise RuntimeError(f"{name}: Tensor must be on device!")
    return fn(input_tensor)


def gelu(input_tensor: Tensor, *, memory_config=None) -> Tensor:
    return _unary("ttnn.gelu", ttl.tensor.gelu, input_tensor)


def relu(input_tensor: Tensor, *, memory_config=None) -> Tensor:
    return _unary("ttnn.relu", ttl.tensor.relu, input_tensor)


def silu(input_tensor: Tensor, *, memory_config=None) -> Tensor:
    return _unary("ttnn.silu", ttl.tensor.silu, input_tensor)
