"""ttnn.matmul / ttnn.linear (ttnn/ttnn/operations/matmul.py:295-416,441-516; ttnn/cpp/ttnn/operations/matmul.hpp:44-214).

The validation of the operands (validation.hpp:17-74 through matmul.hpp:39-42), the shape rules and the dispatch are in the
C++ host layer (``_ttmi.ttnn_matmul``); Tensix-only arguments are accepted and ignored here."""
from __future__ import annotations

from typing import Optional, Tuple

from tt_lib.tensor import DataType, Tensor, _handle_or_none, _m, _opt, _wrap


def create_matmul_1d_systolic_array_program_config(*, input_shape_a: Tuple[int, ...], input_shape_b: Tuple[int, ...], core_grid=None,
                                                   activation: Optional[str] = None, fp32_dst: Optional[bool] = False):
    """ttnn/ttnn/operations/matmul.py:82-160: the 1D program config for two shapes.  The per-core tile counts describe a
    Tensix grid and steer nothing here; they are filled in (tiles divided evenly over the cores of the grid) so that code
    which prints or forwards the object keeps working, and the activation is carried as ``fused_activation``."""
    from tt_lib.operations.primary import MatmulMultiCoreReuseMultiCast1DProgramConfig

    _m().activation_code(activation)                    # rejects unknown names with the reference's message
    if core_grid is None:
        import ttnn

        core_grid = ttnn.CoreGrid(y=8, x=8)
    *batch_a, m, k = (int(x) for x in input_shape_a)
    n = int(input_shape_b[-1])
    if int(input_shape_b[-2]) != k:
        raise RuntimeError("The k dimension does not match between tensors")
    tiles = lambda extent: -(-extent // 32)
    rows = tiles(m)
    for extent in batch_a:
        rows *= extent
    cores = core_grid.num_cores
    wide = tiles(n) >= rows
    return MatmulMultiCoreReuseMultiCast1DProgramConfig(
        compute_with_storage_grid_size=(core_grid.x, core_grid.y), in0_block_w=1, out_subblock_h=1, out_subblock_w=1,
        per_core_M=rows if wide else -(-rows // cores), per_core_N=-(-tiles(n) // cores) if wide else tiles(n), fuse_batch=True,
        fused_activation=activation, mcast_in0=wide)


def _activation_of(program_config, activation):
    """The activation a call asks for: its own argument, else the one its program config carries."""
    if activation is not None or program_config is None:
        return activation
    fused = getattr(program_config, "fused_activation", None)
    if fused is None or isinstance(fused, str):
        return fused
    from tt_lib.tensor import FusibleActivation, FusibleActivationWithParam

    if not isinstance(fused, FusibleActivationWithParam):
        fused = FusibleActivationWithParam(fused)
    return {FusibleActivation.GELU: "gelu", FusibleActivation.RELU: "relu", FusibleActivation.SILU: "silu"}[fused.op_type]


def _run(operation_name, a, b, bias, activation, dtype):
    for t, name in ((a, "input_tensor_a"), (b, "input_tensor_b")) + (((bias, "bias"),) if bias is not None else ()):
        if not isinstance(t, Tensor):
            raise RuntimeError(f"{operation_name}: {name} must be a ttnn.Tensor")
    return _wrap(_m().ttnn_matmul(operation_name, a._t, b._t, _handle_or_none(bias), activation, _opt(dtype)))


def matmul(input_tensor_a: Tensor, input_tensor_b: Tensor, *, memory_config=None, dtype: Optional[DataType] = None,
           core_grid=None, program_config=None, use_1d_systolic_array: Optional[bool] = None, compute_kernel_config=None) -> Tensor:
    """C = A @ B, B's batch dimensions either all 1 (broadcast) or equal to A's.  Output: bfloat16, TILE layout, on device."""
    return _run("ttnn.matmul", input_tensor_a, input_tensor_b, None, _activation_of(program_config, None), dtype)


def linear(input_tensor_a: Tensor, input_tensor_b: Tensor, *, bias: Optional[Tensor] = None, memory_config=None,
           dtype: Optional[DataType] = None, core_grid=None, program_config=None, activation: Optional[str] = None,
           use_1d_systolic_array: Optional[bool] = None, compute_kernel_config=None) -> Tensor:
    """act(A @ B + bias): bias row-broadcast, activation in {None, "relu", "gelu", "silu"}, fused into the GEMM epilogue."""
    return _run("ttnn.linear", input_tensor_a, input_tensor_b, bias, _activation_of(program_config, activation), dtype)


def gated_linear(input_tensor_a: Tensor, gate_weight: Tensor, up_weight: Tensor, *, activation: Optional[str] = "silu",
                 memory_config=None, dtype: Optional[DataType] = None, core_grid=None, compute_kernel_config=None) -> Tensor:
    """act(A @ W_gate) * (A @ W_up) in ONE launch.  No counterpart in tt-metal, whose gated MLPs issue
    ``ttnn.linear(x, w1, activation="silu")``, ``ttnn.linear(x, w3)`` and ``ttnn.mul``
    (models/demos/mistral7b/tt/mistral_mlp.py:43-82); exported as ``ttnn.experimental.gated_linear``.  Both weight tensors are
    block-float, of one dtype and shape, and stream through the same workgroups, which share the activation loads."""
    for t, name in ((input_tensor_a, "input_tensor_a"), (gate_weight, "gate_weight"), (up_weight, "up_weight")):
        if not isinstance(t, Tensor):
            raise RuntimeError(f"ttnn.experimental.gated_linear: {name} must be a ttnn.Tensor")
    act = _m().activation_code(activation)
    return _wrap(_m().matmul_gated(input_tensor_a._t, gate_weight._t, up_weight._t, act, _opt(dtype), "ttnn.experimental.gated_linear"))
