"""``tt_lib.operations.primary.matmul`` (tt_eager/tt_lib/csrc/operations/primary/module.hpp:217-300)."""
from __future__ import annotations

from ttmi import capi

from .. import tensor as _t

_ACT = {None: capi.ACT_NONE, "relu": capi.ACT_RELU, "gelu": capi.ACT_GELU, "silu": capi.ACT_SILU}


def matmul(input_tensor_a, input_tensor_b, bias=None, program_config=None, output_mem_config=None, output_dtype=None,
           compute_kernel_config=None, untilize_out=False, *, activation=None):
    """Mixed dtype (bf16 activations x block-float weights) is legal here (bmm_op.cpp:839).  program_config and
    compute_kernel_config describe Tensix grids and fidelity phases and are accepted and ignored; a fused activation
    carried by the program config (`fused_activation`) is honoured, and so is untilize_out (a ROW_MAJOR bfloat16 output:
    bmm_op.cpp:1069, checks at :536-538 and :865-867)."""
    fused = activation if activation is not None else getattr(program_config, "fused_activation", None)
    if isinstance(fused, (tuple, list)):
        fused = fused[0]
    if fused is not None and not isinstance(fused, str):
        fused = getattr(fused, "name", str(fused)).lower()
    if fused not in _ACT:
        raise RuntimeError(f"{fused} is not supported as activation function")
    batch_b = 1
    for extent in tuple(input_tensor_b.shape.with_tile_padding())[:-2]:
        batch_b *= extent
    return _t._matmul(input_tensor_a, input_tensor_b, bcast_batch=batch_b == 1, bias=bias, activation=_ACT[fused],
                      output_dtype=output_dtype, op="primary.matmul", untilize_out=untilize_out)
