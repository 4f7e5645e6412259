"""ttnn.from_torch / to_torch / to_layout / to_device / from_device / reshape / clone / __getitem__ (ttnn/ttnn/operations/core.py).

Signature shims: the work — padding rules, conversion sequences, validation of tensors, dispatch to the C ABI — is done by the
C++ host layer in ``_ttmi`` (tt-metal_amd/csrc/host/tensor_ops.cpp); what stays here is what the reference also does in
Python (argument normalisation on torch tensors, slicing the result to the logical shape)."""
from __future__ import annotations

from typing import Optional, Tuple, Union

import torch

import ttnn
from tt_lib.tensor import DataType, Layout, Tensor, Device, _BFP, _as_torch, _m, _opt, _wrap


def _check_rank(operation_name, shape, ranks=(1, 2, 3, 4, 5, 6, 7, 8)):
    if len(shape) not in ranks:
        raise RuntimeError(f"{operation_name}: ttnn.Tensor must be of rank {ranks}, but got {len(shape)}")


def from_torch(tensor: "torch.Tensor", dtype: Optional[DataType] = None, *, layout: Optional[Layout] = ttnn.ROW_MAJOR_LAYOUT,
               device: Optional[Device] = None, memory_config=None, mesh_mapper=None) -> Tensor:
    """core.py:245-311.  For bfloat8_b / bfloat4_b the reference pads to tile multiples, packs, unpacks, tilizes and
    packs again on the host; here that whole sequence is ONE fused kernel (pad + tilize + pack), bit-identical to it."""
    _check_rank("ttnn.from_torch", tensor.shape)
    if tensor.dtype not in (torch.bfloat16, torch.float32, torch.int16, torch.int32, torch.int64, torch.float16):
        raise RuntimeError(f"ttnn.from_torch: ttnn.Tensor must be of type bfloat16/float32/int16/int32/int64/float16, but got {tensor.dtype}")
    if mesh_mapper is not None:
        raise RuntimeError("ttnn.from_torch: mesh_mapper needs several devices; this build drives one GPU")
    if memory_config is not None and device is None:
        raise RuntimeError("device must be specified when memory_config is specified")
    if dtype in _BFP:
        if len(tensor.shape) < 2:
            raise RuntimeError("ttnn.from_torch: bfloat8_b/bfloat4_b requires at least 2 dimensions!")
        if layout != ttnn.TILE_LAYOUT:
            raise RuntimeError("ttnn.from_torch: bfloat8_b/bfloat4_b requires TILE_LAYOUT!")
        src = tensor
        if src.dtype == torch.float16:
            src = src.to(torch.bfloat16)          # the reference's dtype-less pre-pass rounds fp16 to bf16 (core.py:282)
        if src.dtype not in (torch.float32, torch.bfloat16):
            src = src.to(torch.float32)
        src = src.contiguous().cpu()
        src_dtype = DataType.FLOAT32 if src.dtype == torch.float32 else DataType.BFLOAT16
        return _wrap(_m().ttnn_from_torch_block_float(src.data_ptr(), int(src_dtype), list(src.shape), int(dtype),
                                                      device.device_id if device is not None else -1))
    t = Tensor(tensor, dtype)
    if layout is not None:
        t = to_layout(t, layout)
    if device is not None:
        t = to_device(t, device, memory_config=memory_config or ttnn.DRAM_MEMORY_CONFIG)
    return t


def to_torch(tensor: Tensor, *, torch_rank: Optional[int] = None, mesh_composer=None) -> "torch.Tensor":
    """core.py:336-394: block-float tensors come back as float32, sliced to the logical shape."""
    if mesh_composer is not None:
        raise RuntimeError("ttnn.to_torch: mesh_composer needs several devices; this build drives one GPU")
    logical = tuple(tensor._shape)
    _check_rank("ttnn.to_torch", logical)
    out = _as_torch(_m().ttnn_to_torch(tensor._t))
    out = out[tuple(slice(None, x) for x in logical)]
    if torch_rank is None:
        return out
    while len(out.shape) != torch_rank:
        if out.shape[0] != 1:
            raise RuntimeError("ttnn: Unable to squeeze to desired rank!")
        out = out.squeeze(0)
    return out


def to_layout(tensor: Tensor, layout: Layout, dtype: Optional[DataType] = None, memory_config=None, use_multicore: bool = False) -> Tensor:
    """core.py:609-803: TILE pads the last two dimensions to multiples of 32 with zeros and keeps the logical shape."""
    if layout not in (ttnn.ROW_MAJOR_LAYOUT, ttnn.TILE_LAYOUT):
        raise RuntimeError(f"Unsupported layout: {layout}")
    return _wrap(_m().ttnn_to_layout(tensor._t, int(layout), _opt(dtype)))


def to_device(tensor: Tensor, device: Device, *, memory_config=None) -> Tensor:
    return tensor.to(device)


def from_device(tensor: Tensor) -> Tensor:
    return tensor.cpu()


def deallocate(tensor: Tensor) -> None:
    tensor.deallocate(force=True)


def reshape(input_tensor: Tensor, shape: Union["ttnn.Shape", Tuple[int, ...]]) -> Tensor:
    return input_tensor.reshape(shape)


def unsqueeze_to_4D(tensor: Tensor) -> Tensor:
    rank = len(tensor._shape)
    if rank == 4:
        return tensor
    if rank > 4:
        raise RuntimeError("Tensor cannot have more than 4 dimensions!")
    lead = (1,) * (4 - rank)
    return tensor.reshape(ttnn.Shape(lead + tuple(tensor._shape), lead + tuple(tensor._padded)))


def clone(tensor: Tensor, memory_config=None, dtype: Optional[DataType] = None) -> Tensor:
    """core.py:819-839: a copy of a device tensor, optionally in another dtype; the layout stays."""
    if not isinstance(tensor, Tensor) or not ttnn.is_tensor_storage_on_device(tensor):
        raise RuntimeError("ttnn.clone: Tensor must be on device!")
    return _wrap(_m().clone(tensor._t, _opt(dtype)))


def _getitem(input_tensor: Tensor, slices) -> Tensor:
    """ttnn.Tensor.__getitem__ (core.py:56-114).  As in the reference, only prefixes of a device tensor of rank <= 4 can be
    taken (any non-zero start raises, core.py:95-97); in TILE layout the `unpad` behind it copies whole tiles up to the
    tile-rounded end and the logical shape is set by a reshape, so block-float tiles keep their bytes."""
    input_rank = len(input_tensor._shape)
    if isinstance(slices, int):
        slices = (slice(None, slices, None),)
    elif isinstance(slices, slice):
        slices = (slices,)
    elif slices is Ellipsis:
        raise RuntimeError("Ellipsis is not supported!")
    normalized = []
    for s in slices:
        if isinstance(s, int):
            normalized.append(slice(None, s, None))
        elif isinstance(s, slice):
            normalized.append(s)
        else:
            raise RuntimeError("Invalid slice type!")
    if len(normalized) > input_rank:
        raise RuntimeError(f"Too many slices for tensor of rank {input_rank}")
    normalized += [slice(None, None, None)] * (input_rank - len(normalized))
    if not (ttnn.is_tensor_storage_on_device(input_tensor) and input_rank <= 4):
        raise RuntimeError("ttnn.Tensor.__getitem__: cannot slice the given tensor on the device!")
    t4 = unsqueeze_to_4D(input_tensor)
    normalized = [slice(None, None, None)] * (4 - input_rank) + normalized
    for s in normalized:
        if s.start not in (None, 0) or s.step not in (None, 1):
            raise RuntimeError("ttnn.Tensor.__getitem__: cannot slice the given tensor on the device!")
    end = [s.stop if s.stop is not None else t4._shape[i] for i, s in enumerate(normalized)]
    for e in end:
        if e < 0:
            raise RuntimeError("ttnn.Tensor.__getitem__: slice end outside the tensor")
    out = _wrap(_m().ttnn_getitem_prefix(t4._t, [int(e) for e in end]))
    return out.reshape(ttnn.Shape(tuple(out._shape)[-input_rank:], tuple(out._padded)[-input_rank:]))


Tensor.__getitem__ = _getitem
