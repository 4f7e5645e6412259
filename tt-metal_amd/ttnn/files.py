"""ttnn.dump_tensor / load_tensor / as_tensor (ttnn/ttnn/operations/core.py:869-980): tensors as files in the reference's
own format (tt_eager/tensor/serialization.cpp:86-141), so that a weight cache written by either side loads on the other."""
from __future__ import annotations

import pathlib
from typing import Optional, Union

import ttnn
import tt_lib as ttl
from tt_lib.tensor import DataType, Device, Layout, Tensor


def load_tensor(file_name: Union[str, pathlib.Path]) -> Tensor:
    file_name = pathlib.Path(file_name)
    if not file_name.exists():
        raise RuntimeError(f"Unable to load the tensor from {file_name}.  The file does not exist.")     # core.py:876-877
    if not file_name.is_file():
        raise RuntimeError(f"Unable to load the tensor from {file_name}.  The file is not a file.")      # core.py:878-879
    return ttl.tensor.load_tensor(str(file_name))


def dump_tensor(file_name: Union[str, pathlib.Path], tensor: Tensor) -> None:
    if not isinstance(tensor, Tensor):
        raise RuntimeError("ttnn.dump_tensor: expected a ttnn.Tensor")
    ttl.tensor.dump_tensor(str(pathlib.Path(file_name)), tensor)


def as_tensor(tensor: "torch.Tensor", dtype: Optional[DataType] = None, *, layout: Optional[Layout] = ttnn.ROW_MAJOR_LAYOUT,
              device: Optional[Device] = None, memory_config=None, cache_file_name: Optional[Union[str, pathlib.Path]] = None) -> Tensor:
    """from_torch, or — with cache_file_name — the tensor file `<name>_dtype_<D>_layout_<L>.bin` if it loads, else
    from_torch followed by writing that file (core.py:922-980)."""
    import torch

    if len(tensor.shape) not in (1, 2, 3, 4, 5, 6, 7, 8):
        raise RuntimeError(f"ttnn.as_tensor: ttnn.Tensor must be of rank (1, 2, 3, 4, 5, 6, 7, 8), but got {len(tensor.shape)}")
    dtypes = (torch.bfloat16, torch.float32, torch.int16, torch.int32, torch.int64, torch.float16)
    if tensor.dtype not in dtypes:
        raise RuntimeError(f"ttnn.as_tensor: ttnn.Tensor must be of type {dtypes}, but got {tensor.dtype}")
    if cache_file_name is None:
        return ttnn.from_torch(tensor, dtype=dtype, layout=layout, device=device, memory_config=memory_config)
    dtype_name = dtype.name if dtype is not None else "None"
    layout_name = layout.name if layout is not None else "None"
    cache_file_name = f"{cache_file_name}_dtype_{dtype_name}_layout_{layout_name}.bin"
    try:
        loaded = load_tensor(cache_file_name)
    except (FileNotFoundError, RuntimeError):
        loaded = ttnn.from_torch(tensor, dtype=dtype, layout=layout)
        pathlib.Path(cache_file_name).parent.mkdir(parents=True, exist_ok=True)
        dump_tensor(cache_file_name, loaded)
    if device is None:
        return loaded
    return ttnn.to_device(loaded, device, memory_config=memory_config)


def get_memory_config(tensor: Tensor):
    return getattr(tensor, "_mem_config", None) or ttnn.DRAM_MEMORY_CONFIG
