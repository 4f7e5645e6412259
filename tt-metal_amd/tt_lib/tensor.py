"""``tt_lib.tensor`` for the block-float path: DataType / Layout / StorageType, Tensor, matmul, bmm, pad / unpad, ...

A signature shim over the C++ host layer in the pybind11 module ``_ttmi`` (tt-metal_amd/csrc/host/tensor_ops.cpp), which
holds the Tensor object, the shape and padding rules, the argument validation and the dispatch to the C ABI
(include/ttmi.h) — the split the reference has between tt_lib (Python names) and tt_lib._C
(tt_eager/tt_lib/csrc/tt_lib_bindings_tensor_pytensor.cpp:746-1300, tt_lib_bindings_tensor_custom_bmm_ops.cpp:50-81).
torch provides memory (its allocator) and the stream; it computes nothing on device data.  Host-storage tensors keep their
bytes in CPU memory exactly as the reference lays them out (packed uint32 words for block-float), device-storage tensors
in HBM.
"""
from __future__ import annotations

import enum
from typing import Optional

import torch

from ttmi import capi, pybind


class DataType(enum.IntEnum):  # tt_eager/tensor/types.hpp:26-34
    BFLOAT16 = 0
    FLOAT32 = 1
    UINT32 = 2
    BFLOAT8_B = 3
    BFLOAT4_B = 4
    UINT16 = 6
    INVALID = 7


class Layout(enum.IntEnum):  # tt_eager/tensor/types.hpp:24
    ROW_MAJOR = 0
    TILE = 1
    INVALID = 2


class StorageType(enum.IntEnum):  # tt_eager/tensor/types.hpp:36-41
    OWNED = 0
    DEVICE = 1
    BORROWED = 2
    MULTI_DEVICE = 3


class BufferType(enum.IntEnum):
    DRAM = 0
    L1 = 1


class TensorMemoryLayout(enum.IntEnum):
    INTERLEAVED = 0
    SINGLE_BANK = 1
    HEIGHT_SHARDED = 2
    WIDTH_SHARDED = 3
    BLOCK_SHARDED = 4


class MathFidelity(enum.IntEnum):
    LoFi = 0
    HiFi2 = 2
    HiFi3 = 3
    HiFi4 = 4


class MemoryConfig:
    """Accepted for signature compatibility; every buffer lives in HBM."""

    def __init__(self, memory_layout=TensorMemoryLayout.INTERLEAVED, buffer_type=BufferType.DRAM, shard_spec=None):
        self.memory_layout, self.buffer_type, self.shard_spec = memory_layout, buffer_type, shard_spec

    def __eq__(self, other):
        return isinstance(other, MemoryConfig) and (self.memory_layout, self.buffer_type) == (other.memory_layout, other.buffer_type)

    def __repr__(self):
        return f"MemoryConfig({self.memory_layout.name}, {self.buffer_type.name})"


_modules = {}
_module_name = "_ttmi"


def use_test_library(on: bool) -> None:
    """Tests only: the mirror runs on _ttmi_test / libttmi_test.so (the build with the ttmi_test_* hooks) until switched back.
    Tensors made under one of the two do not pass to the other."""
    global _module_name
    _module_name = "_ttmi_test" if on else "_ttmi"
    capi.use_test_library(on)


def _m():
    """The C++ host layer, with torch installed as its runtime: memory from torch's allocator (flat uint8 tensors own every
    buffer), launches on torch's current stream."""
    if _module_name not in _modules:
        capi.lib()                                     # fail loudly when the HIP library is not built
        mod = pybind.module(_module_name)

        def allocate(nbytes, device):
            if device < 0:
                return torch.empty(nbytes, dtype=torch.uint8)
            return torch.empty(nbytes, dtype=torch.uint8, device=torch.device("cuda", device))

        mod.set_runtime(allocate, lambda device: torch.cuda.current_stream(device).cuda_stream, torch.cuda.is_available)
        _modules[_module_name] = mod
    return _modules[_module_name]


class Device:
    """One MI355X.  tt_lib.device.CreateDevice(id) in the reference opens a Tensix chip; here it selects a HIP device."""

    def __init__(self, device_id: int = 0):
        capi.lib()  # fail loudly when the HIP library is not built
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU visible: the block-float path has no CPU fallback")
        self.device_id = device_id
        self.torch_device = torch.device("cuda", device_id)

    def id(self):
        return self.device_id

    def __eq__(self, other):
        return isinstance(other, Device) and other.device_id == self.device_id

    def __hash__(self):
        return hash(("ttmi.Device", self.device_id))

    def __repr__(self):
        return f"Device(id={self.device_id}, MI355X)"


_BFP = (DataType.BFLOAT8_B, DataType.BFLOAT4_B)
_TORCH = {DataType.BFLOAT16: torch.bfloat16, DataType.FLOAT32: torch.float32, DataType.UINT32: torch.int32, DataType.UINT16: torch.int16,
          DataType.BFLOAT8_B: torch.int32, DataType.BFLOAT4_B: torch.int32}


def _pad32(x: int) -> int:
    return (x + 31) // 32 * 32


def _opt(dtype):
    return None if dtype is None else int(DataType(dtype))


class Tensor:
    """Eager tensor: legacy shape (with tile padding), dtype, layout, storage — a handle on the C++ Tensor of ``_ttmi``.

    Buffer conventions (identical to the reference's byte layout):
      ROW_MAJOR bf16/fp32/ints   dense elements of the padded shape
      TILE      bf16/fp32/ints   32x32 tiles of four 16x16 faces (test_tiles.hpp:24-65)
      block-float                uint32 words; TILE = packed tiles of the tilized tensor, ROW_MAJOR = the
                                 row-major data packed in consecutive 1024-element chunks
                                 (tt_lib_bindings_tensor_pytensor.cpp:145-151)
    """

    def __init__(self, data, data_type: Optional[DataType] = None, device: Optional[Device] = None,
                 layout: Optional[Layout] = None, mem_config: Optional[MemoryConfig] = None, *, _raw=None, _handle=None):
        if _handle is not None:
            self._t = _handle
            return
        if _raw is not None:      # (torch buffer, logical shape, padded shape, dtype, layout, device): memory that torch already holds
            buf, shape, padded, dtype, lay, dev = _raw
            storage = buf.contiguous().reshape(-1).view(torch.uint8)
            self._t = _m().wrap(storage, storage.data_ptr(), storage.numel(), storage.device.index if storage.is_cuda else -1,
                                list(shape), list(padded), int(dtype), int(lay))
            return
        if not isinstance(data, torch.Tensor):
            raise RuntimeError("tt_lib.tensor.Tensor: expected a torch.Tensor")
        t = data.contiguous().cpu()
        if data_type is None:  # pytensor.cpp:38-62
            data_type = {torch.float32: DataType.FLOAT32, torch.float16: DataType.BFLOAT16, torch.bfloat16: DataType.BFLOAT16,
                         torch.int16: DataType.UINT16, torch.int32: DataType.UINT32, torch.int64: DataType.UINT32}.get(t.dtype)
            if data_type is None:
                raise RuntimeError(f"Unsupported DataType: {t.dtype}")
        data_type = DataType(data_type)
        # the host tensor in the storage type of its data type (fp32 for block-float: pytensor.cpp:78-85); the C++ side packs
        src = t.to(torch.float32 if data_type in _BFP else _TORCH[data_type]).contiguous()
        self._t = _m().from_host(src.data_ptr(), list(src.shape), int(data_type))
        if layout is not None and Layout(layout) != Layout.ROW_MAJOR:
            self._t = _m().to_layout(self._t, int(Layout(layout)))
        if device is not None:
            self._t = _m().to_device(self._t, device.device_id)

    # ---- metadata -----------------------------------------------------------------------------------
    @property
    def _shape(self):
        return tuple(self._t.shape)

    @property
    def _padded(self):
        return tuple(self._t.padded_shape)

    @property
    def _dtype(self):
        return DataType(self._t.dtype)

    @property
    def _layout(self):
        return Layout(self._t.layout)

    @property
    def _device(self):
        return Device(self._t.device) if self._t.device >= 0 else None

    @property
    def _buf(self):
        """The buffer as a torch tensor of the storage element type (dense ROW_MAJOR data in the padded shape, else flat)."""
        elements = self._t.storage[:self._t.nbytes].view(_TORCH[self._dtype])
        if self._layout == Layout.ROW_MAJOR and self._dtype not in _BFP:
            return elements.view(self._padded)
        return elements

    @property
    def shape(self):
        import ttnn

        return ttnn.Shape(self._shape, self._padded)

    def get_legacy_shape(self):
        return self.shape.with_tile_padding()

    def shape_without_padding(self):
        return self._shape

    @property
    def dtype(self):
        return self._dtype

    def get_dtype(self):
        return self._dtype

    @property
    def layout(self):
        return self._layout

    def get_layout(self):
        return self._layout

    def storage_type(self):
        # block-float tensors always own a copy (tests/tt_eager/.../test_tensor.py:55-57)
        return StorageType.DEVICE if self._t.device >= 0 else StorageType.OWNED

    def device(self):
        return self._device

    def is_allocated(self):
        return self._t is not None

    def deallocate(self, force: bool = False):
        self._t = None

    def volume(self):
        return self._t.volume()

    def __repr__(self):
        return f"Tensor(shape={self.shape}, dtype={self._dtype.name}, layout={self._layout.name}, storage={self.storage_type().name})"

    # ---- movement -----------------------------------------------------------------------------------
    def to(self, target, mem_config: Optional[MemoryConfig] = None):
        if isinstance(target, Device):
            return _wrap(_m().to_device(self._t, target.device_id))
        return _wrap(_m().to_layout(self._t, int(Layout(target))))

    def cpu(self, blocking: bool = True):
        return _wrap(_m().to_host(self._t))

    def reshape(self, *shape):
        if len(shape) == 1 and not isinstance(shape[0], int):
            shape = shape[0]
        import ttnn

        if isinstance(shape, ttnn.Shape):
            logical, padded = list(shape), list(shape.with_tile_padding())
        else:
            logical = padded = [int(s) for s in shape]
        return _wrap(_m().reshape(self._t, logical, padded))

    # ---- pad / unpad on the host (tt_eager/tensor/tensor.cpp:204-260) ----------------------------------------
    def pad(self, output_tensor_shape, input_tensor_start, pad_value: float):
        return _wrap(_m().pad(self._t, [int(x) for x in output_tensor_shape], [int(x) for x in input_tensor_start], float(pad_value)))

    def unpad(self, output_tensor_start, output_tensor_end):
        return _wrap(_m().unpad(self._t, [int(x) for x in output_tensor_start], [int(x) for x in output_tensor_end]))

    def pad_to_tile(self, pad_value: float):
        return _wrap(_m().pad_to_tile(self._t, float(pad_value)))

    def unpad_from_tile(self, output_tensor_shape):
        return _wrap(_m().unpad_from_tile(self._t, [int(x) for x in output_tensor_shape]))

    def to_torch(self):
        """pytensor.cpp:354-412: block-float comes back as float32 (sequential unpack), others in their own dtype."""
        return _as_torch(_m().to_torch(self._t))


def _wrap(handle) -> Tensor:
    return Tensor(None, _handle=handle)


def _as_torch(host_handle) -> "torch.Tensor":
    """A host tensor of the C++ layer as a torch tensor of its padded shape (the memory is torch's own already)."""
    dtype = _TORCH[DataType(host_handle.dtype)]
    return host_handle.storage[:host_handle.nbytes].view(dtype).view(tuple(host_handle.padded_shape))


def _handle_or_none(t):
    return None if t is None else t._t


def matmul(input_a: Tensor, input_b: Tensor, output_mem_config: Optional[MemoryConfig] = None, kernel_config=None,
           untilize_out: bool = False) -> Tensor:
    """tt_lib.tensor.matmul: [B, C, M, K] x [1, 1, K, N] (tt_lib_bindings_tensor_custom_bmm_ops.cpp:50-65, bmm_op.hpp:388)."""
    return _matmul(input_a, input_b, bcast_batch=True, op="matmul", untilize_out=untilize_out)


def bmm(input_a: Tensor, input_b: Tensor, output_mem_config: Optional[MemoryConfig] = None, kernel_config=None,
        untilize_out: bool = False) -> Tensor:
    """tt_lib.tensor.bmm: [B, C, M, K] x [B, C, K, N] (tt_lib_bindings_tensor_custom_bmm_ops.cpp:66-81, bmm_op.hpp:425)."""
    return _matmul(input_a, input_b, bcast_batch=False, op="bmm", untilize_out=untilize_out)


def _matmul(a: Tensor, b: Tensor, *, bcast_batch: bool, bias: Optional[Tensor] = None, activation: int = capi.ACT_NONE,
            output_dtype: Optional[DataType] = None, op: str = "matmul", untilize_out: bool = False) -> Tensor:
    """Shared body of matmul / bmm / primary.matmul: validation (bmm_op.cpp:518-539,828-1049) and dispatch are in the C++ layer.
    untilize_out: the output is ROW_MAJOR instead of TILE (bmm_op.cpp:1069), bfloat16 only (bmm_op.cpp:536-538, 865-867)."""
    return _wrap(_m().matmul(a._t, b._t, bcast_batch, _handle_or_none(bias), int(activation), _opt(output_dtype), op, bool(untilize_out)))


def unpad(input_tensor: Tensor, output_tensor_start, output_tensor_end, output_mem_config: Optional[MemoryConfig] = None) -> Tensor:
    """tt_lib.tensor.unpad on a device tensor (tt_eager/tt_dnn/op_library/unpad/unpad_op.cpp:95-125): in TILE layout start and
    extent are whole tiles, so tiles are moved as they are and a block-float tensor keeps its codes."""
    return _wrap(_m().device_unpad(input_tensor._t, [int(x) for x in output_tensor_start], [int(x) for x in output_tensor_end]))


# ---- the BERT-Large matmuls (bmm_op.cpp:631-742): fixed shapes, otherwise primary::matmul ----------------------------
def _expect_shape(t: Tensor, shape) -> None:
    if tuple(t._padded) != tuple(shape):
        raise RuntimeError(f"TT_FATAL: Unsupported input shape (expected {list(shape)}, got {list(t._padded)})")


def bert_large_fused_qkv_matmul(input_a: Tensor, input_b: Tensor, bias: Optional[Tensor] = None,
                                output_mem_config: Optional[MemoryConfig] = None, output_dtype: Optional[DataType] = None) -> Tensor:
    """bmm_op.cpp:634-651: [B, 1, 384, 1024] x [1, 1, 1024, 3072]."""
    _expect_shape(input_a, (input_a._padded[0], 1, 384, 1024))
    _expect_shape(input_b, (1, 1, 1024, 3072))
    return _matmul(input_a, input_b, bcast_batch=True, bias=bias, output_dtype=output_dtype, op="bert_large_fused_qkv_matmul")


def bert_large_ff1_matmul(input_a: Tensor, input_b: Tensor, bias: Optional[Tensor] = None, fused_activation=None,
                          output_mem_config: Optional[MemoryConfig] = None, output_dtype: Optional[DataType] = None) -> Tensor:
    """bmm_op.cpp:653-672: [B, 1, 384, 1024] x [1, 1, 1024, 4096], optional fused activation (the L1 / DRAM rule of :656 is
    about Tensix buffers and has nothing to check here)."""
    _expect_shape(input_a, (input_a._padded[0], 1, 384, 1024))
    _expect_shape(input_b, (1, 1, 1024, 4096))
    return _matmul(input_a, input_b, bcast_batch=True, bias=bias, activation=_fused_activation_code(fused_activation),
                   output_dtype=output_dtype, op="bert_large_ff1_matmul")


def bert_large_ff2_matmul(input_a: Tensor, input_b: Tensor, bias: Optional[Tensor] = None,
                          output_mem_config: Optional[MemoryConfig] = None, output_dtype: Optional[DataType] = None) -> Tensor:
    """bmm_op.cpp:674-691: [B, 1, 384, 4096] x [1, 1, 4096, 1024]."""
    _expect_shape(input_a, (input_a._padded[0], 1, 384, 4096))
    _expect_shape(input_b, (1, 1, 4096, 1024))
    return _matmul(input_a, input_b, bcast_batch=True, bias=bias, output_dtype=output_dtype, op="bert_large_ff2_matmul")


def bert_large_selfout_matmul(input_a: Tensor, input_b: Tensor, bias: Optional[Tensor] = None,
                              output_mem_config: Optional[MemoryConfig] = None, output_dtype: Optional[DataType] = None) -> Tensor:
    """bmm_op.cpp:693-710: [B, 1, 384, 1024] x [1, 1, 1024, 1024]."""
    _expect_shape(input_a, (input_a._padded[0], 1, 384, 1024))
    _expect_shape(input_b, (1, 1, 1024, 1024))
    return _matmul(input_a, input_b, bcast_batch=True, bias=bias, output_dtype=output_dtype, op="bert_large_selfout_matmul")


def bert_large_pre_softmax_bmm(input_a: Tensor, input_b: Tensor, output_mem_config: Optional[MemoryConfig] = None,
                               output_dtype: Optional[DataType] = None) -> Tensor:
    """bmm_op.cpp:712-726: [B, 16, 384, 64] x [B, 16, 64, 384], every slice with its own right operand."""
    b = input_a._padded[0]
    _expect_shape(input_a, (b, 16, 384, 64))
    _expect_shape(input_b, (b, 16, 64, 384))
    return _matmul(input_a, input_b, bcast_batch=False, output_dtype=output_dtype, op="bert_large_pre_softmax_bmm")


def bert_large_post_softmax_bmm(input_a: Tensor, input_b: Tensor, output_mem_config: Optional[MemoryConfig] = None,
                                output_dtype: Optional[DataType] = None) -> Tensor:
    """bmm_op.cpp:728-742: [B, 16, 384, 384] x [B, 16, 384, 64]."""
    b = input_a._padded[0]
    _expect_shape(input_a, (b, 16, 384, 384))
    _expect_shape(input_b, (b, 16, 384, 64))
    return _matmul(input_a, input_b, bcast_batch=False, output_dtype=output_dtype, op="bert_large_post_softmax_bmm")


# ---- compute kernel configs (tt_lib_bindings_tensor.cpp:325-348) ----------------------------------------------------
class GrayskullComputeKernelConfig:
    """Fidelity phases of the Tensix matrix unit: nothing of it applies here (the GEMMs multiply exact bf16 operands and add in
    fp32 whatever it says); model code constructs it and passes it as ``compute_kernel_config``, so the object exists."""

    def __init__(self, *, math_fidelity=None, math_approx_mode: bool = True):
        self.math_fidelity, self.math_approx_mode = math_fidelity, math_approx_mode


class WormholeComputeKernelConfig:
    def __init__(self, *, math_fidelity=None, math_approx_mode: bool = True, fp32_dest_acc_en: bool = False, packer_l1_acc: bool = False):
        self.math_fidelity, self.math_approx_mode = math_fidelity, math_approx_mode
        self.fp32_dest_acc_en, self.packer_l1_acc = fp32_dest_acc_en, packer_l1_acc


# ---- fused activations and the Falcon matmuls (bmm_op.cpp:747-807) -------------------------------------------------
class FusibleActivation(enum.IntEnum):  # UnaryOpType, tt_eager/tt_dnn/op_library/eltwise_unary/eltwise_unary_op.hpp:17-78
    GELU = 2
    RELU = 3
    SILU = 48


class FusibleActivationWithParam:
    """UnaryWithParam (tt_lib_bindings_tensor.cpp:113-128): an activation and its parameter; for GELU the parameter selects the
    Tensix fast-and-approximate mode, which has no counterpart here (the exact erf form is used either way)."""

    def __init__(self, op_type, param: float = 0.0):
        if isinstance(op_type, (tuple, list)):
            op_type, param = op_type[0], (op_type[1] if len(op_type) > 1 else 0.0)
        self.op_type, self.param = FusibleActivation(op_type), float(param)


_FUSED = {FusibleActivation.GELU: capi.ACT_GELU, FusibleActivation.RELU: capi.ACT_RELU, FusibleActivation.SILU: capi.ACT_SILU}


def _fused_activation_code(fused_activation) -> int:
    if fused_activation is None:
        return capi.ACT_NONE
    if not isinstance(fused_activation, FusibleActivationWithParam):
        fused_activation = FusibleActivationWithParam(fused_activation)
    return _FUSED[fused_activation.op_type]


def falcon_fused_qkv_matmul(input_a: Tensor, input_b: Tensor, bias: Optional[Tensor] = None,
                            output_mem_config: Optional[MemoryConfig] = None, output_dtype: Optional[DataType] = None) -> Tensor:
    """bmm_op.cpp:747-750: A x B with B broadcast over the batch."""
    return _matmul(input_a, input_b, bcast_batch=True, bias=bias, output_dtype=output_dtype, op="falcon_fused_qkv_matmul")


def falcon_selfout_matmul(input_a: Tensor, input_b: Tensor, bias: Optional[Tensor] = None,
                          output_mem_config: Optional[MemoryConfig] = None, output_dtype: Optional[DataType] = None) -> Tensor:
    """bmm_op.cpp:752-755."""
    return _matmul(input_a, input_b, bcast_batch=True, bias=bias, output_dtype=output_dtype, op="falcon_selfout_matmul")


def falcon_dense_4h_to_h_matmul(input_a: Tensor, input_b: Tensor, bias: Optional[Tensor] = None,
                                output_mem_config: Optional[MemoryConfig] = None, output_dtype: Optional[DataType] = None,
                                packer_l1_acc: Optional[bool] = None) -> Tensor:
    """bmm_op.cpp:757-771 (packer_l1_acc is a Tensix accumulation mode: accepted, without effect)."""
    return _matmul(input_a, input_b, bcast_batch=True, bias=bias, output_dtype=output_dtype, op="falcon_dense_4h_to_h_matmul")


def falcon_dense_h_to_4h_matmul(input_a: Tensor, input_b: Tensor, bias: Optional[Tensor] = None, fused_activation=None,
                                output_mem_config: Optional[MemoryConfig] = None, output_dtype: Optional[DataType] = None) -> Tensor:
    """bmm_op.cpp:773-791: above 1024 rows the reference accepts only [1, 1, seq, 4544] x [1, 1, 4544, 18176] without a
    fused activation; the same conditions are rejected here."""
    seq_len = input_a._padded[-2]
    if seq_len > 1024:
        if fused_activation is not None:
            raise RuntimeError("TT_FATAL: not fused_activation.has_value()")
        if seq_len % 32:
            raise RuntimeError("TT_FATAL: Falcon mm's seq_len must be a multiple of 32!")
        if tuple(input_a._padded) != (1, 1, seq_len, 4544) or tuple(input_b._padded) != (1, 1, 4544, 18176):
            raise RuntimeError("TT_FATAL: Unsupported input shape")
    return _matmul(input_a, input_b, bcast_batch=True, bias=bias, activation=_fused_activation_code(fused_activation),
                   output_dtype=output_dtype, op="falcon_dense_h_to_4h_matmul")


def falcon_lm_head_matmul(input_a: Tensor, input_b: Tensor, bias: Optional[Tensor] = None,
                          output_mem_config: Optional[MemoryConfig] = None, output_dtype: Optional[DataType] = None) -> Tensor:
    """bmm_op.cpp:793-807."""
    return _matmul(input_a, input_b, bcast_batch=True, bias=bias, output_dtype=output_dtype, op="falcon_lm_head_matmul")


# ---- elementwise (eltwise_binary_op.hpp:108-140, eltwise_unary_op.hpp) ----------------------------------------------
def _eltwise(op: int, a: Tensor, b=None, scalar: float = 0.0, name: str = "eltwise") -> Tensor:
    return _wrap(_m().eltwise(op, a._t, _handle_or_none(b), float(scalar), name))


def add(input_a: Tensor, input_b: Tensor, output_mem_config: Optional[MemoryConfig] = None) -> Tensor:
    return _eltwise(capi.OP_ADD, input_a, input_b, name="add")


def sub(input_a: Tensor, input_b: Tensor, output_mem_config: Optional[MemoryConfig] = None) -> Tensor:
    return _eltwise(capi.OP_SUB, input_a, input_b, name="sub")


def mul(input_a: Tensor, input_b: Tensor, output_mem_config: Optional[MemoryConfig] = None) -> Tensor:
    return _eltwise(capi.OP_MUL, input_a, input_b, name="mul")


def add_unary(input_a: Tensor, scalar: float, output_mem_config: Optional[MemoryConfig] = None) -> Tensor:
    return _eltwise(capi.OP_ADD, input_a, None, scalar, name="add_unary")


def mul_unary(input_a: Tensor, scalar: float, output_mem_config: Optional[MemoryConfig] = None) -> Tensor:
    return _eltwise(capi.OP_MUL, input_a, None, scalar, name="mul_unary")


def gelu(input_a: Tensor, fast_and_approx: bool = True, output_mem_config: Optional[MemoryConfig] = None) -> Tensor:
    return _eltwise(capi.OP_GELU, input_a, name="gelu")


def relu(input_a: Tensor, output_mem_config: Optional[MemoryConfig] = None) -> Tensor:
    return _eltwise(capi.OP_RELU, input_a, name="relu")


def silu(input_a: Tensor, output_mem_config: Optional[MemoryConfig] = None) -> Tensor:
    return _eltwise(capi.OP_SILU, input_a, name="silu")


# ---- tensor files (tt_eager/tensor/serialization.cpp:86-141) --------------------------------------------------------
# File = the raw bytes of `Shape` (tt_eager/tensor/types.hpp:46-63,118-121 as the x86-64 System V ABI lays it out), then
# DataType and Layout as 32-bit integers, then the element count as a 64-bit integer and the elements; written and read by
# the C++ layer (FileHeader in csrc/host/tensor_ops.cpp).
def dump_tensor(file_name: str, tensor: Tensor) -> None:
    _m().dump_tensor(str(file_name), tensor._t)


def load_tensor(file_name: str) -> Tensor:
    return _wrap(_m().load_tensor(str(file_name)))


# ---- device-resident dtype changes (tt_eager/tt_dnn/op_library/copy/copy_op.hpp:42-44, tilize/tilize_op.hpp:71-73) -------
# On Tensix the conversion happens in the packer of a data-movement kernel, whose rounding is not stated in the sources at
# hand; here the values pass through the host packers' arithmetic (one pack of the tile-ordered values), which is what
# the reference's own host-side typecast of a block-float tensor does.
def typecast(input_tensor: Tensor, dtype: DataType, output_mem_config: Optional[MemoryConfig] = None) -> Tensor:
    return _wrap(_m().typecast(input_tensor._t, int(DataType(dtype))))


def clone(input_tensor: Tensor, output_mem_config: Optional[MemoryConfig] = None, output_dtype: Optional[DataType] = None) -> Tensor:
    return _wrap(_m().clone(input_tensor._t, _opt(output_dtype)))


def tilize(input_tensor: Tensor, output_mem_config: Optional[MemoryConfig] = None, use_multicore: bool = False,
           output_dtype: Optional[DataType] = None) -> Tensor:
    """tilize_op.hpp:71-73: ROW_MAJOR -> TILE on the device, optionally into another dtype (bf16 -> block-float)."""
    return _wrap(_m().tilize(input_tensor._t, _opt(output_dtype)))
