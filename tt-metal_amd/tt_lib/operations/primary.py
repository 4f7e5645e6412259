"""``tt_lib.operations.primary``: matmul, matmul_1d and the program-config objects they take
(tt_eager/tt_lib/csrc/operations/primary/module.hpp:53-406; tt_eager/tt_dnn/op_library/bmm/bmm_op.hpp:284-346,
bmm_op.cpp:1279-1295)."""
from __future__ import annotations

from ttmi import capi

from .. import tensor as _t

_ACT = {None: capi.ACT_NONE, "relu": capi.ACT_RELU, "gelu": capi.ACT_GELU, "silu": capi.ACT_SILU}


class MatmulProgramConfig:
    """How a Tensix grid runs a matmul.  Nothing of it applies to one GPU, where the library picks the kernel by shape;
    the objects exist so that model code written against tt_lib constructs and passes them unchanged.  The one field that
    changes the result, ``fused_activation``, is honoured."""

    _fields: tuple = ()

    def __init__(self, **kwargs):
        missing = [f for f in self._fields if f not in kwargs]
        unknown = [k for k in kwargs if k not in self._fields]
        if missing or unknown:       # pybind raises TypeError for a call that matches no constructor
            raise TypeError(f"{type(self).__name__}(): incompatible constructor arguments (missing {missing}, unknown {unknown})")
        for name, value in kwargs.items():
            setattr(self, name, value)

    def __repr__(self):
        return f"{type(self).__name__}({', '.join(f'{f}={getattr(self, f)!r}' for f in self._fields)})"


class MatmulDefaultProgramConfig(MatmulProgramConfig):          # module.hpp:56-58
    pass


class MatmulMultiCoreReuseProgramConfig(MatmulProgramConfig):   # module.hpp:60-70
    _fields = ("compute_with_storage_grid_size", "in0_block_w", "out_subblock_h", "out_subblock_w", "per_core_M", "per_core_N")


class MatmulMultiCoreReuseMultiCastProgramConfig(MatmulProgramConfig):     # module.hpp:72-95
    _fields = ("compute_with_storage_grid_size", "in0_block_w", "out_subblock_h", "out_subblock_w", "per_core_M", "per_core_N",
               "transpose_mcast", "fused_activation")


class MatmulMultiCoreReuseMultiCast1DProgramConfig(MatmulProgramConfig):   # module.hpp:97-122
    _fields = ("compute_with_storage_grid_size", "in0_block_w", "out_subblock_h", "out_subblock_w", "per_core_M", "per_core_N",
               "fuse_batch", "fused_activation", "mcast_in0")


def _activation_code(activation, program_config) -> int:
    """An activation name (this mirror's keyword), or what the program config carries: a FusibleActivation, a
    (FusibleActivation, parameter) pair or a FusibleActivationWithParam, as the reference's UnaryWithParam converts from."""
    if activation is not None:
        if activation not in _ACT:
            raise RuntimeError(f"{activation} is not supported as activation function")
        return _ACT[activation]
    fused = getattr(program_config, "fused_activation", None)
    if isinstance(fused, str):
        if fused not in _ACT:
            raise RuntimeError(f"{fused} is not supported as activation function")
        return _ACT[fused]
    try:
        return _t._fused_activation_code(fused)
    except (KeyError, ValueError):
        raise RuntimeError(f"{fused} is not supported as activation function") from None


def _batch_of_b(input_tensor_b) -> int:
    batch_b = 1
    for extent in tuple(input_tensor_b.shape.with_tile_padding())[:-2]:
        batch_b *= extent
    return batch_b


def matmul(input_tensor_a, input_tensor_b, bias=None, program_config=None, output_mem_config=None, output_dtype=None,
           compute_kernel_config=None, untilize_out=False, *, activation=None):
    """Mixed dtype (bf16 activations x block-float weights) is legal here (bmm_op.cpp:839).  program_config and
    compute_kernel_config describe Tensix grids and fidelity phases and are accepted and ignored; a fused activation
    carried by the program config (`fused_activation`) is honoured, and so is untilize_out (a ROW_MAJOR bfloat16 output:
    bmm_op.cpp:1069, checks at :536-538 and :865-867)."""
    return _t._matmul(input_tensor_a, input_tensor_b, bcast_batch=_batch_of_b(input_tensor_b) == 1, bias=bias,
                      activation=_activation_code(activation, program_config), output_dtype=output_dtype, op="primary.matmul",
                      untilize_out=untilize_out)


def matmul_1d(input_tensor_a, input_tensor_b, *, bias=None, program_config=None, output_mem_config=None, output_dtype=None,
              compute_kernel_config=None):
    """module.hpp:373-406: primary.matmul with a MatmulMultiCoreReuseMultiCast1DProgramConfig, which the reference derives from
    the shapes when none is passed (bmm_op.cpp:1289-1295); Falcon-40B's MLP issues its GEMMs this way
    (models/demos/falcon40b/tt/falcon_mlp.py:97-135)."""
    return _t._matmul(input_tensor_a, input_tensor_b, bcast_batch=_batch_of_b(input_tensor_b) == 1, bias=bias,
                      activation=_activation_code(None, program_config), output_dtype=output_dtype, op="primary.matmul_1d")
