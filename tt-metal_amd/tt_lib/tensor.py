"""``tt_lib.tensor`` for the block-float path: DataType / Layout / StorageType, Tensor, matmul, bmm.

Mirrors the pybind surface of tt_eager/tt_lib/csrc/tt_lib_bindings_tensor_pytensor.cpp:746-1300 and
tt_lib_bindings_tensor_custom_bmm_ops.cpp:50-81.  Every conversion and the matmul run as HIP kernels behind
the C ABI (include/ttmi.h); torch only carries memory.  Host-storage tensors keep their bytes in CPU memory
exactly as the reference lays them out (packed uint32 words for block-float), device-storage tensors in HBM.
"""
from __future__ import annotations

import enum
import struct
from typing import Optional, Sequence

import torch

from ttmi import capi


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

    def __repr__(self):
        return f"Device(id={self.device_id}, MI355X)"


_BFP = (DataType.BFLOAT8_B, DataType.BFLOAT4_B)
_TORCH = {DataType.BFLOAT16: torch.bfloat16, DataType.FLOAT32: torch.float32, DataType.UINT32: torch.int32, DataType.UINT16: torch.int16}


def _pad32(x: int) -> int:
    return (x + 31) // 32 * 32


def _run_on_gpu(buf: torch.Tensor, fn, device: Optional[torch.device] = None):
    """Runs fn(cuda tensor) -> cuda tensor; host buffers are staged through the GPU and copied back."""
    if buf.is_cuda:
        return fn(buf)
    capi.lib()
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU visible: block-float conversions run as HIP kernels and have no CPU fallback")
    return fn(buf.to(device or "cuda")).cpu()


class Tensor:
    """Eager tensor: legacy shape (with tile padding), dtype, layout, storage.

    Buffer conventions (identical to the reference's byte layout):
      ROW_MAJOR bf16/fp32/ints   dense torch tensor of the padded shape
      TILE      bf16/fp32/ints   flat torch tensor, 32x32 tiles of four 16x16 faces (test_tiles.hpp:24-65)
      block-float                flat int32 words; TILE = packed tiles of the tilized tensor, ROW_MAJOR = the
                                 row-major data packed in consecutive 1024-element chunks
                                 (tt_lib_bindings_tensor_pytensor.cpp:145-151)
    """

    def __init__(self, data, data_type: Optional[DataType] = None, device: Optional[Device] = None,
                 layout: Optional[Layout] = None, mem_config: Optional[MemoryConfig] = None, *, _raw=None):
        if _raw is not None:
            self._buf, self._shape, self._padded, self._dtype, self._layout, self._device = _raw
            return
        if not isinstance(data, torch.Tensor):
            raise RuntimeError("tt_lib.tensor.Tensor: expected a torch.Tensor")
        t = data.contiguous()
        if data_type is None:  # pytensor.cpp:38-62
            data_type = {torch.float32: DataType.FLOAT32, torch.float16: DataType.BFLOAT16, torch.bfloat16: DataType.BFLOAT16,
                         torch.int16: DataType.UINT16, torch.int32: DataType.UINT32, torch.int64: DataType.UINT32}.get(t.dtype)
            if data_type is None:
                raise RuntimeError(f"Unsupported DataType: {t.dtype}")
        data_type = DataType(data_type)
        self._shape = tuple(int(s) for s in t.shape)
        self._padded = self._shape
        self._dtype, self._layout, self._device = data_type, Layout.ROW_MAJOR, None
        if data_type in _BFP:  # pytensor.cpp:78-85,145-157: cast to fp32, pack sequential 1024-chunks, declare ROW_MAJOR
            if t.numel() % 1024:
                raise RuntimeError("TT_ASSERT: fp32_vec.size() % num_float_in_tile == 0 (block-float tensors hold whole tiles)")
            src = t.to(torch.float32).reshape(-1)
            self._buf = _run_on_gpu(src, lambda d: capi.pack_chunks(int(data_type), d, False))
        else:
            self._buf = t.to(_TORCH[data_type]).clone()
        if layout is not None and Layout(layout) != Layout.ROW_MAJOR:
            converted = self.to(Layout(layout))
            self._buf, self._padded, self._layout = converted._buf, converted._padded, converted._layout
        if device is not None:
            self._buf, self._device = self._buf.to(device.torch_device), device

    # ---- metadata -----------------------------------------------------------------------------------
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
        return StorageType.DEVICE if self._device is not None else StorageType.OWNED

    def device(self):
        return self._device

    def is_allocated(self):
        return self._buf is not None

    def deallocate(self, force: bool = False):
        self._buf = None

    def volume(self):
        v = 1
        for s in self._padded:
            v *= s
        return v

    def __repr__(self):
        return f"Tensor(shape={self.shape}, dtype={self._dtype.name}, layout={self._layout.name}, storage={self.storage_type().name})"

    def _like(self, buf, shape=None, padded=None, dtype=None, layout=None, device="keep"):
        return Tensor(None, _raw=(buf, shape if shape is not None else self._shape, padded if padded is not None else self._padded,
                                  dtype if dtype is not None else self._dtype, layout if layout is not None else self._layout,
                                  self._device if device == "keep" else device))

    # ---- movement -----------------------------------------------------------------------------------
    def to(self, target, mem_config: Optional[MemoryConfig] = None):
        if isinstance(target, Device):
            return self._like(self._buf.to(target.torch_device), device=target)
        target = Layout(target)
        if target == self._layout:
            return self
        batch, h, w = self._bhw(self._padded)
        dev = self._device.torch_device if self._device else None
        if target == Layout.TILE:
            if self._padded[-1] % 32 or (len(self._padded) > 1 and self._padded[-2] % 32):
                raise RuntimeError("TT_ASSERT: Unsupported shape for tensor conversion (height and width must be multiples of 32)")
            if self._dtype in _BFP:  # tensor_impl.cpp:179-197: unpack -> tilize as fp32 -> pack
                fmt = int(self._dtype)
                fn = lambda d: capi.pack_chunks(fmt, capi.tilize(capi.unpack_chunks(fmt, d, False).view(batch, h, w)), False)
            else:
                fn = lambda d: capi.tilize(d.view(batch, h, w))
            return self._like(_run_on_gpu(self._buf, fn, dev), layout=Layout.TILE)
        if self._dtype in _BFP:
            fmt = int(self._dtype)
            fn = lambda d: capi.pack_chunks(fmt, capi.untilize(capi.unpack_chunks(fmt, d, False), (batch, h, w)).reshape(-1), False)
            return self._like(_run_on_gpu(self._buf, fn, dev), layout=Layout.ROW_MAJOR)
        fn = lambda d: capi.untilize(d, (batch, h, w)).view(self._padded)
        return self._like(_run_on_gpu(self._buf, fn, dev), layout=Layout.ROW_MAJOR)

    def cpu(self, blocking: bool = True):
        return self._like(self._buf.cpu(), device=None)

    def reshape(self, *shape):
        if len(shape) == 1 and not isinstance(shape[0], int):
            shape = shape[0]
        import ttnn

        if isinstance(shape, ttnn.Shape):
            logical, padded = tuple(shape), tuple(shape.with_tile_padding())
        else:
            logical = padded = tuple(int(s) for s in shape)
        v = 1
        for s in padded:
            v *= s
        if v != self.volume():
            raise RuntimeError(f"TT_ASSERT: reshape changes the volume ({self.volume()} -> {v})")
        buf = self._buf
        if self._layout == Layout.ROW_MAJOR and self._dtype not in _BFP:
            buf = buf.reshape(padded)
        elif self._layout == Layout.TILE and (padded[-2:] != self._padded[-2:]):
            raise RuntimeError("reshape of a TILE tensor must keep the last two padded dimensions")
        return self._like(buf, shape=logical, padded=padded)

    # ---- pad / unpad on the host (tt_eager/tensor/tensor.cpp:204-260) ----------------------------------------
    def _window(self, dst_shape, offset, fill, what):
        """dst[i] = self[i - offset] inside self, `fill` elsewhere: pad<T> / unpad<T> (tensor_impl.hpp:508-660), and for
        block-float tensors unpack -> fp32 pad / unpad -> pack (tensor_impl.cpp:200-283) in one kernel."""
        if self._device is not None:
            raise RuntimeError("TT_THROW: Device storage isn't supported")          # tensor_impl.hpp:590, 675
        if self._layout != Layout.ROW_MAJOR:
            raise RuntimeError(f"TT_ASSERT: Tensor layout must be ROW_MAJOR for {what}")
        if len(self._padded) != 4 or len(dst_shape) != 4:
            raise RuntimeError(f"{what}: shapes must have rank 4")
        dst_shape = tuple(int(x) for x in dst_shape)
        code = int(self._dtype)
        if self._dtype in _BFP:
            volume = dst_shape[0] * dst_shape[1] * dst_shape[2] * dst_shape[3]
            if volume % 1024:
                raise RuntimeError("TT_ASSERT: fp32_vec.size() % num_float_in_tile == 0 (block-float tensors hold whole tiles)")
            src = self._buf
        else:
            src = self._buf.view(self._padded)
        return _run_on_gpu(src, lambda d: capi.copy_window(code, d, self._padded, dst_shape, offset, fill))

    def pad(self, output_tensor_shape, input_tensor_start, pad_value: float):
        """tensor.cpp:204-224: the tensor placed at input_tensor_start inside a tensor of output_tensor_shape filled with pad_value."""
        out_shape = tuple(int(x) for x in output_tensor_shape)
        start = tuple(int(x) for x in input_tensor_start)
        if len(out_shape) != 4 or len(start) != 4 or len(self._padded) != 4:
            raise RuntimeError("pad: shapes must have rank 4")
        for i in range(4):
            if self._padded[i] + start[i] > out_shape[i]:      # tensor_impl.hpp:522-525
                raise RuntimeError(f"TT_ASSERT: input_tensor_shape[{i}] + input_tensor_start[{i}] <= output_tensor_shape[{i}]")
        buf = self._window(out_shape, start, float(pad_value), "padding")
        return self._like(buf, shape=tuple(self._padded), padded=out_shape)

    def unpad(self, output_tensor_start, output_tensor_end):
        """tensor.cpp:226-230: the elements output_tensor_start..output_tensor_end (inclusive in every dimension)."""
        start = tuple(int(x) for x in output_tensor_start)
        end = tuple(int(x) for x in output_tensor_end)
        if len(start) != 4 or len(end) != 4 or len(self._padded) != 4:
            raise RuntimeError("unpad: shapes must have rank 4")
        for i in range(4):                                      # tensor_impl.hpp:614-627
            if start[i] >= self._padded[i] or end[i] >= self._padded[i] or start[i] > end[i]:
                raise RuntimeError(f"TT_ASSERT: output_tensor_start[{i}] <= output_tensor_end[{i}] < input_tensor_shape[{i}]")
        out_shape = tuple(e - b + 1 for b, e in zip(start, end))
        buf = self._window(out_shape, tuple(-b for b in start), 0.0, "unpadding")
        return self._like(buf, shape=out_shape, padded=out_shape)

    def pad_to_tile(self, pad_value: float):
        """tensor.cpp:232-246: height and width rounded up to 32, the tensor in the top left corner."""
        if len(self._padded) != 4:
            raise RuntimeError("pad_to_tile: the tensor must have rank 4")
        n, c, h, w = self._padded
        return self.pad((n, c, _pad32(h), _pad32(w)), (0, 0, 0, 0), pad_value)

    def unpad_from_tile(self, output_tensor_shape):
        """tensor.cpp:248-260: the inverse of pad_to_tile for a given logical shape."""
        out = tuple(int(x) for x in output_tensor_shape)
        if len(out) != 4 or len(self._padded) != 4:
            raise RuntimeError("unpad_from_tile: shapes must have rank 4")
        if self._padded[0] != out[0] or self._padded[1] != out[1]:
            raise RuntimeError("TT_ASSERT: Input shape must match output shape apart from last 2 dims")
        if self._padded[2] % 32 or self._padded[3] % 32:
            raise RuntimeError("TT_ASSERT: Last 2 dims of input shape must be multiples of 32")
        if not (self._padded[2] - 32 < out[2] <= self._padded[2] and self._padded[3] - 32 < out[3] <= self._padded[3]):
            raise RuntimeError("TT_ASSERT: Last 2 dims of output must be within range to have been padded to input")
        return self.unpad((0, 0, 0, 0), tuple(x - 1 for x in out))

    def to_torch(self):
        """pytensor.cpp:354-412: block-float comes back as float32 (sequential unpack), others in their own dtype."""
        if self._device is not None:
            raise RuntimeError("Tensor must be on host to be converted to torch (call .cpu() first)")
        if self._dtype in _BFP:
            fmt = int(self._dtype)
            return _run_on_gpu(self._buf, lambda d: capi.unpack_chunks(fmt, d, False)).view(self._padded)
        if self._layout == Layout.TILE:
            return self._buf.clone().view(self._padded)
        return self._buf.clone().view(self._padded)

    @staticmethod
    def _bhw(shape):
        shape = tuple(shape)
        if len(shape) > 4:
            raise RuntimeError(f"Rank {len(shape)} is not supported!")  # tensor_impl.hpp:143-155
        h = shape[-2] if len(shape) > 1 else 1
        w = shape[-1]
        batch = 1
        for s in shape[:-2]:
            batch *= s
        return batch, h, w


def _matmul(a: Tensor, b: Tensor, *, bcast_batch: bool, bias: Optional[Tensor] = None, activation: int = capi.ACT_NONE,
            output_dtype: Optional[DataType] = None, op: str = "matmul") -> Tensor:
    """Shared body of matmul / bmm / primary.matmul (validation of bmm_op.cpp:518-539,828-1049)."""
    for t, name in ((a, "input_tensor_a"), (b, "input_tensor_b")):
        if t.storage_type() != StorageType.DEVICE:
            raise RuntimeError(f"TT_FATAL: Operands to {op} need to be on device! ({name})")
        if t.layout != Layout.TILE:
            raise RuntimeError(f"TT_FATAL: Inputs to {op} must be tilized ({name})")
    pa, pb = tuple(a._padded), tuple(b._padded)
    if len(pa) < 2 or len(pb) < 2 or len(pa) > 4 or len(pb) > 4:
        raise RuntimeError(f"TT_FATAL: {op} supports ranks 2 to 4")
    if pa[-1] != pb[-2]:
        raise RuntimeError("TT_FATAL: The width of the first tensor must be equal to the height of the second tensor "
                           f"(a.shape[-1] = {pa[-1]}, b.shape[-2] = {pb[-2]})")
    if b.dtype not in _BFP:
        raise RuntimeError(f"{op}: this build accelerates block-float weights (BFLOAT8_B / BFLOAT4_B); got {b.dtype.name}")
    if a.dtype not in (DataType.BFLOAT16, DataType.BFLOAT8_B, DataType.BFLOAT4_B):
        raise RuntimeError(f"TT_FATAL: Unsupported data format for input a: {a.dtype.name}")  # bmm_op.cpp:839
    batch_a = 1
    for s in pa[:-2]:
        batch_a *= s
    batch_b = 1
    for s in pb[:-2]:
        batch_b *= s
    if bcast_batch:
        if batch_b != 1:
            raise RuntimeError("TT_FATAL: matmul (batch bcast variant) expects input tensors of shapes BCMK*11KN=BCMN")  # bmm_op.cpp:529
    elif batch_b != batch_a:
        raise RuntimeError("TT_FATAL: bmm (non-bcast matmul) expects input tensors of shapes BCMK*BCKN=BCMN")  # bmm_op.cpp:533
    m, k, n = pa[-2], pa[-1], pb[-1]
    a_buf = a._buf
    bias_buf = None
    if bias is not None:
        if bias.storage_type() != StorageType.DEVICE:
            raise RuntimeError("TT_FATAL: bias must be on device")
        if bias._padded[-1] != n:
            raise RuntimeError("TT_FATAL: bias width must match the output width")
        bb = bias
        bh = bb._padded[-2] if len(bb._padded) > 1 else 1
        # bias is a [.., 32, N] tile row in the reference; row 0 carries the values (matmul.hpp:117-140)
        if bb.dtype not in (DataType.BFLOAT16,) + _BFP:
            raise RuntimeError(f"TT_FATAL: Unsupported data format for the bias: {bb.dtype.name}")
        with torch.cuda.device(a._device.torch_device):
            if bb.dtype in _BFP:
                row = capi.unpack_tensor(int(bb.dtype), bb._buf, (1, bh, n), dtype=torch.bfloat16)
            elif bb.layout == Layout.TILE:
                row = capi.untilize(bb._buf, (1, bh, n))
            else:
                row = bb._buf.view(-1, n)
            bias_buf = row.reshape(-1, n)[0].contiguous()      # the first of the tile's 32 rows
    out_dtype = DataType(output_dtype) if output_dtype is not None else a.dtype  # bmm_op.hpp:388: output takes input a's dtype
    if out_dtype not in (DataType.BFLOAT16,) + _BFP:
        raise RuntimeError(f"{op}: output dtype {out_dtype.name} is not supported (BFLOAT16, BFLOAT8_B, BFLOAT4_B)")
    with torch.cuda.device(a._device.torch_device):
        if a.dtype in _BFP:   # block-float activations: expanded (exactly) to bf16 tiles by one kernel in front of the GEMM
            a_buf = capi.typecast_tiles(a._buf, int(a.dtype), capi.BFLOAT16)
        c = capi.matmul_bfp(a_buf, capi.TILE, b._buf, int(b.dtype), batch_a, batch_b, m, k, n, bias=bias_buf,
                            activation=activation, c_layout=capi.TILE, out_dtype=torch.bfloat16)
        if out_dtype in _BFP:  # the packer of the reference's compute kernel, applied to the bf16 result tiles by one kernel
            c = capi.typecast_tiles(c, capi.BFLOAT16, int(out_dtype))
    logical = tuple(a._shape[:-1]) + (b._shape[-1],)
    padded = pa[:-1] + (n,)
    return Tensor(None, _raw=(c, logical, padded, out_dtype, Layout.TILE, a._device))


def matmul(input_a: Tensor, input_b: Tensor, output_mem_config: Optional[MemoryConfig] = None, kernel_config=None,
           untilize_out: bool = False) -> Tensor:
    """tt_lib.tensor.matmul: [B, C, M, K] x [1, 1, K, N] (tt_lib_bindings_tensor_custom_bmm_ops.cpp:50-65, bmm_op.hpp:388)."""
    return _matmul(input_a, input_b, bcast_batch=True, op="matmul")


def bmm(input_a: Tensor, input_b: Tensor, output_mem_config: Optional[MemoryConfig] = None, kernel_config=None,
        untilize_out: bool = False) -> Tensor:
    """tt_lib.tensor.bmm: [B, C, M, K] x [B, C, K, N] (tt_lib_bindings_tensor_custom_bmm_ops.cpp:66-81, bmm_op.hpp:425)."""
    return _matmul(input_a, input_b, bcast_batch=False, op="bmm")


def unpad(input_tensor: Tensor, output_tensor_start, output_tensor_end, output_mem_config: Optional[MemoryConfig] = None) -> Tensor:
    """tt_lib.tensor.unpad on a device tensor (tt_eager/tt_dnn/op_library/unpad/unpad_op.cpp:95-125): in TILE layout start and
    extent are whole tiles, so tiles are moved as they are and a block-float tensor keeps its codes."""
    if input_tensor.storage_type() != StorageType.DEVICE:
        raise RuntimeError("TT_FATAL: Operands to unpad need to be on device!")
    padded = tuple(input_tensor._padded)
    start, end = tuple(int(x) for x in output_tensor_start), tuple(int(x) for x in output_tensor_end)
    if len(padded) != 4 or len(start) != 4 or len(end) != 4:
        raise RuntimeError("unpad: shapes must have rank 4")
    for i in range(4):
        if start[i] >= padded[i] or end[i] >= padded[i] or start[i] > end[i]:
            raise RuntimeError(f"TT_FATAL: output_tensor_start[{i}] <= output_tensor_end[{i}] < input shape[{i}]")
    out_shape = tuple(e - b + 1 for b, e in zip(start, end))
    with torch.cuda.device(input_tensor._device.torch_device):
        if input_tensor.layout == Layout.TILE:
            if out_shape[-2] % 32 or start[-2] % 32 or out_shape[-1] % 32 or start[-1] % 32:
                raise RuntimeError("TT_FATAL: Can only unpad tilized tensor with full tiles")
            grid = lambda sh: (sh[0], sh[1], sh[2] // 32, sh[3] // 32)
            buf = capi.unpad_tiles(int(input_tensor.dtype), input_tensor._buf, grid(padded), grid(start), grid(out_shape))
        else:
            if input_tensor.dtype in _BFP:
                raise RuntimeError("TT_FATAL: block-float tensors on device are in TILE layout")
            elem = input_tensor._buf.element_size()
            if (out_shape[-1] * elem) % 4 or (start[-1] * elem) % 4:
                raise RuntimeError("TT_FATAL: RM unpadding requires output X size to be packable")
            buf = capi.copy_window(int(input_tensor.dtype), input_tensor._buf.view(padded), padded, out_shape, tuple(-b for b in start))
    return input_tensor._like(buf, shape=out_shape, padded=out_shape)


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
def _as_bf16_buffer(t: Tensor) -> "torch.Tensor":
    """Flat bf16 device buffer in the tensor's own element order; block-float operands are expanded (exactly)."""
    if t.storage_type() != StorageType.DEVICE:
        raise RuntimeError("TT_FATAL: Operands to eltwise ops need to be on device!")
    if t.dtype in _BFP:
        return capi.typecast_tiles(t._buf, int(t.dtype), capi.BFLOAT16)     # same element order, <= 7 significant bits: exact
    if t.dtype != DataType.BFLOAT16:
        raise RuntimeError(f"TT_FATAL: Unsupported data format {t.dtype.name} (BFLOAT16, BFLOAT8_B, BFLOAT4_B)")
    return t._buf.reshape(-1)


def _eltwise(op: int, a: Tensor, b=None, scalar: float = 0.0, name: str = "eltwise") -> Tensor:
    if b is not None:
        if tuple(a._padded) != tuple(b._padded):
            raise RuntimeError(f"TT_FATAL: {name}: input shapes must be the same ({tuple(a._padded)} vs {tuple(b._padded)}); "
                               "broadcast forms are not part of this build")
        if a.layout != b.layout:
            raise RuntimeError(f"TT_FATAL: {name}: inputs must have the same layout")
    with torch.cuda.device(a._device.torch_device):
        out = capi.eltwise(op, _as_bf16_buffer(a), _as_bf16_buffer(b) if b is not None else None, scalar)
        if a.dtype in _BFP:      # output takes input a's dtype (eltwise_binary_op.hpp:124-126)
            out = capi.typecast_tiles(out, capi.BFLOAT16, int(a.dtype))
        elif a.layout == Layout.ROW_MAJOR:
            out = out.view(a._padded)
    return a._like(out)


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
# DataType and Layout as 32-bit integers, then the element count as a 64-bit integer and the elements:
#   offset   0  u64      Shape::rank_
#            8  u32 x 8  Shape::dimensions_ (the shape WITH padding; unused entries 0)
#           40  u64      Padding::rank_
#           48  {u64 front, u64 back} x 8   Padding::pad_dimensions_ (back = padded - logical size)
#          176  i32      Padding::pad_value_ (PadValue::Any = 0), 4 bytes of struct padding
#          184  i32      DataType          188  i32  Layout
#          192  u64      number of elements (uint32 words for block-float and UINT32, 2-byte elements for BFLOAT16 / UINT16)
#          200  elements
_FILE_HEADER = struct.Struct("<Q8IQ16QiiiiQ")
_FILE_ELEMENT = {DataType.BFLOAT16: torch.bfloat16, DataType.UINT16: torch.int16, DataType.FLOAT32: torch.float32,
                 DataType.UINT32: torch.int32, DataType.BFLOAT8_B: torch.int32, DataType.BFLOAT4_B: torch.int32}


def dump_tensor(file_name: str, tensor: Tensor) -> None:
    if tensor.storage_type() == StorageType.DEVICE:
        raise RuntimeError("TT_THROW: Device storage isn't supported")     # serialization.cpp:113-115
    rank = len(tensor._padded)
    if rank > 8:
        raise RuntimeError("TT_THROW: Shape supports up to 8 dimensions")
    dims = list(tensor._padded) + [0] * (8 - rank)
    pads = []
    for i in range(8):
        pads += [0, (tensor._padded[i] - tensor._shape[i]) if i < rank else 0]
    flat = tensor._buf.contiguous().reshape(-1)
    header = _FILE_HEADER.pack(rank, *dims, rank, *pads, 0, 0, int(tensor.dtype), int(tensor.layout), flat.numel())
    assert len(header) == 200
    with open(file_name, "wb") as f:
        f.write(header)
        f.write(flat.view(torch.uint8).numpy().tobytes())


def load_tensor(file_name: str) -> Tensor:
    try:
        f = open(file_name, "rb")
    except OSError:
        raise RuntimeError(f'Cannot open "{file_name}"')                 # serialization.cpp:122-125
    with f:
        raw = f.read(200)
        if len(raw) != 200:
            raise RuntimeError(f'"{file_name}" is too short to hold a tensor header')
        fields = _FILE_HEADER.unpack(raw)
        rank, dims, pads = fields[0], fields[1:9], fields[10:26]
        dtype, layout, count = DataType(fields[28]), Layout(fields[29]), fields[30]
        if rank > 8 or dtype not in _FILE_ELEMENT:
            raise RuntimeError("TT_THROW: Unsupported DataType")
        elem = _FILE_ELEMENT[dtype]
        nbytes = count * torch.empty(0, dtype=elem).element_size()
        payload = f.read(nbytes)
        if len(payload) != nbytes:
            raise RuntimeError(f'"{file_name}" ends inside the tensor data')
    padded = tuple(int(d) for d in dims[:rank])
    logical = tuple(int(d) - int(pads[2 * i]) - int(pads[2 * i + 1]) for i, d in enumerate(padded))
    buf = torch.frombuffer(bytearray(payload), dtype=torch.uint8).view(elem)
    if layout == Layout.ROW_MAJOR and dtype not in _BFP:
        buf = buf.view(padded)
    return Tensor(None, _raw=(buf, logical, padded, dtype, layout, None))


# ---- device-resident dtype changes (tt_eager/tt_dnn/op_library/copy/copy_op.hpp:42-44, tilize/tilize_op.hpp:71-73) -------
# On Tensix the conversion happens in the packer of a data-movement kernel, whose rounding is not stated in the sources at
# hand; here the values pass through the host packers' arithmetic (one pack of the tile-ordered values), which is what
# the reference's own host-side typecast of a block-float tensor does.
def typecast(input_tensor: Tensor, dtype: DataType, output_mem_config: Optional[MemoryConfig] = None) -> Tensor:
    dtype = DataType(dtype)
    if input_tensor.storage_type() != StorageType.DEVICE:
        raise RuntimeError("TT_FATAL: Operands to copy need to be on device!")
    if dtype == input_tensor.dtype:
        return input_tensor._like(input_tensor._buf.clone())
    floats = (DataType.BFLOAT16, DataType.FLOAT32) + _BFP
    if input_tensor.dtype not in floats or dtype not in floats:
        raise RuntimeError(f"TT_FATAL: typecast between {input_tensor.dtype.name} and {dtype.name} is not supported")
    if (input_tensor.dtype in _BFP or dtype in _BFP) and input_tensor.layout != Layout.TILE:
        raise RuntimeError("TT_FATAL: block-float tensors on device are in TILE layout")
    with torch.cuda.device(input_tensor._device.torch_device):
        src, src_dtype = input_tensor._buf, int(input_tensor.dtype)
        if input_tensor.dtype in _BFP and dtype in _BFP:        # through bf16, which holds every block-float value exactly
            src, src_dtype = capi.typecast_tiles(src, src_dtype, capi.BFLOAT16), capi.BFLOAT16
        if input_tensor.layout == Layout.ROW_MAJOR:
            # dense row-major floats: the element order does not matter to a bf16 <-> fp32 conversion; whole "tiles" of
            # 1024 elements are what the entry point counts in, so the tail is padded for the call and cut off again
            flat = src.reshape(-1)
            pad = (-flat.numel()) % 1024
            if pad:
                flat = torch.cat([flat, flat.new_zeros(pad)])
            out = capi.typecast_tiles(flat, src_dtype, int(dtype))[:flat.numel() - pad].view(input_tensor._padded)
        else:
            out = capi.typecast_tiles(src, src_dtype, int(dtype))
    return input_tensor._like(out, dtype=dtype)


def clone(input_tensor: Tensor, output_mem_config: Optional[MemoryConfig] = None, output_dtype: Optional[DataType] = None) -> Tensor:
    if output_dtype is None or DataType(output_dtype) == input_tensor.dtype:
        if input_tensor.storage_type() != StorageType.DEVICE:
            raise RuntimeError("TT_FATAL: Operands to copy need to be on device!")
        return input_tensor._like(input_tensor._buf.clone())
    return typecast(input_tensor, output_dtype, output_mem_config)


def tilize(input_tensor: Tensor, output_mem_config: Optional[MemoryConfig] = None, use_multicore: bool = False,
           output_dtype: Optional[DataType] = None) -> Tensor:
    """tilize_op.hpp:71-73: ROW_MAJOR -> TILE on the device, optionally into another dtype (bf16 -> block-float)."""
    if input_tensor.storage_type() != StorageType.DEVICE:
        raise RuntimeError("TT_FATAL: Operands to tilize need to be on device!")
    if input_tensor.layout != Layout.ROW_MAJOR:
        raise RuntimeError("TT_FATAL: Can only tilize row major data")
    if input_tensor._padded[-1] % 32 or (len(input_tensor._padded) > 1 and input_tensor._padded[-2] % 32):
        raise RuntimeError("TT_FATAL: tilize needs height and width to be multiples of 32")
    tiles = input_tensor.to(Layout.TILE)
    if output_dtype is None or DataType(output_dtype) == tiles.dtype:
        return tiles
    return typecast(tiles, output_dtype, output_mem_config)
