"""ttnn.from_torch / to_torch / to_layout / to_device / from_device / reshape (ttnn/ttnn/operations/core.py)."""
from __future__ import annotations

from typing import Optional, Tuple, Union

import torch

import ttnn
import tt_lib.tensor as ttl_tensor
from tt_lib.tensor import DataType, Layout, Tensor, Device, _BFP, _TORCH, _pad32, _run_on_gpu
from ttmi import capi


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
        if len(tensor.shape) > 4:
            raise RuntimeError(f"Rank {len(tensor.shape)} is not supported!")  # tensor_impl.hpp:143-155
        src = tensor
        if src.dtype == torch.float16:
            src = src.to(torch.bfloat16)          # the reference's dtype-less pre-pass rounds fp16 to bf16 (core.py:282)
        if src.dtype not in (torch.float32, torch.bfloat16):
            src = src.to(torch.float32)
        src = src.contiguous()
        logical = tuple(src.shape)
        padded = logical[:-2] + (_pad32(logical[-2]), _pad32(logical[-1]))
        fmt = int(dtype)
        if device is not None:
            # the source goes to the device once and the packed words stay there
            with torch.cuda.device(device.torch_device):
                words = capi.pack_tensor(fmt, src.to(device.torch_device))
        else:
            words = _run_on_gpu(src, lambda d: capi.pack_tensor(fmt, d))
        return Tensor(None, _raw=(words, logical, padded, DataType(dtype), Layout.TILE, device))

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
    _check_rank("ttnn.to_torch", tensor._shape)
    logical, padded = tuple(tensor._shape), tuple(tensor._padded)
    if tensor.dtype in _BFP and tensor.layout == Layout.TILE:
        fmt = int(tensor.dtype)
        batch, h, w = Tensor._bhw(padded)
        # one fused kernel: unpack + untilize, cropping the tile padding of the last two dimensions
        crop = padded[:-2] + (logical[-2], logical[-1])
        out = _run_on_gpu(tensor._buf, lambda d: capi.unpack_tensor(fmt, d, (batch, logical[-2], logical[-1])))
        out = out.cpu().view(crop)
    else:
        host = tensor.cpu() if tensor.storage_type() == ttnn.DEVICE_STORAGE_TYPE else tensor
        if host.layout != Layout.ROW_MAJOR:
            host = host.to(Layout.ROW_MAJOR)
        out = host.to_torch()
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
    if tensor.layout == layout and (dtype is None or dtype == tensor.dtype):
        return tensor
    if dtype is not None and dtype != tensor.dtype:
        # core.py:684-685, 706-711: only on the device and only towards TILE_LAYOUT (tilize with an output dtype)
        if not ttnn.is_tensor_storage_on_device(tensor) or layout != ttnn.TILE_LAYOUT:
            raise RuntimeError(f"Unsupported datatype conversion to {dtype}")
        tiles = to_layout(tensor, layout) if tensor.layout != layout else tensor
        return ttl_tensor.typecast(tiles, dtype)
    if tensor.layout == layout:
        return tensor
    logical, padded = tuple(tensor._shape), tuple(tensor._padded)
    if layout == ttnn.TILE_LAYOUT:
        if tensor.dtype in _BFP:
            return tensor.to(Layout.TILE)
        rank = len(logical)
        if rank < 2 or rank > 4:
            raise RuntimeError(f"Rank {rank} is not supported!")
        batch = 1
        for s in logical[:-2]:
            batch *= s
        dense = tensor._buf.reshape(padded)[tuple(slice(None, x) for x in logical)].reshape(batch, logical[-2], logical[-1])
        dev = tensor._device.torch_device if tensor._device else None
        buf = _run_on_gpu(dense.contiguous(), lambda d: capi.tilize(d), dev)  # pads with zeros and tilizes in one kernel
        new_padded = logical[:-2] + (_pad32(logical[-2]), _pad32(logical[-1]))
        return Tensor(None, _raw=(buf, logical, new_padded, tensor.dtype, Layout.TILE, tensor._device))
    # to ROW_MAJOR: the tile padding stays part of the (padded) shape, as in the reference
    return tensor.to(Layout.ROW_MAJOR)


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
    return ttl_tensor.clone(tensor, output_mem_config=memory_config, output_dtype=dtype)


def _getitem(input_tensor: Tensor, slices) -> Tensor:
    """ttnn.Tensor.__getitem__ (core.py:56-114): prefixes of a device tensor of rank <= 4.  In TILE layout the reference's
    `unpad` copies whole tiles up to the tile-rounded end and the logical shape is set by a reshape, so block-float tiles
    keep their bytes (nothing is re-quantised); the same happens here."""
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
    for i, e in enumerate(end):
        if e < 0 or e > t4._shape[i]:
            raise RuntimeError("ttnn.Tensor.__getitem__: slice end outside the tensor")
    padded_end = list(end)
    if t4.layout == Layout.TILE:
        padded_end[-1], padded_end[-2] = _pad32(end[-1]), _pad32(end[-2])
    full = tuple(t4._padded)
    buf = t4._buf
    if tuple(padded_end) != full:
        if t4.layout == Layout.TILE:
            per_tile = capi.TILE_BYTES[int(t4.dtype)] // buf.element_size()
            tiles = buf.view(full[0], full[1], full[2] // 32, full[3] // 32, per_tile)
            buf = tiles[:padded_end[0], :padded_end[1], :padded_end[2] // 32, :padded_end[3] // 32].contiguous().view(-1)
        else:
            buf = buf.view(full)[:padded_end[0], :padded_end[1], :padded_end[2], :padded_end[3]].contiguous()
    out_shape = tuple(end[-input_rank:])
    out_padded = tuple(padded_end[-input_rank:])
    if t4.layout == Layout.ROW_MAJOR and t4.dtype not in _BFP:
        buf = buf.reshape(out_padded)
    return Tensor(None, _raw=(buf, out_shape, out_padded, t4.dtype, t4.layout, t4._device))


Tensor.__getitem__ = _getitem
