"""Host-side behaviour of the TT-NN / tt_lib mirror that needs no GPU: shapes, names, argument validation.

The cases follow tests/ttnn/unit_tests/test_shape.py and the error paths of ttnn/ttnn/operations/core.py:245-311
and ttnn/ttnn/operations/matmul.py:200-220 of the reference.
"""
import pytest
import torch

import ttnn
import tt_lib


def test_shape_equality_operator():
    a = ttnn.Shape((1, 2, 3, 4))
    assert a == (1, 2, 3, 4) and (1, 2, 3, 4) == a
    assert a.with_tile_padding() == (1, 2, 3, 4) and (1, 2, 3, 4) == a.with_tile_padding()
    b = ttnn.Shape((1, 2, 3, 4))
    assert a == b
    c = ttnn.Shape((1, 2, 3, 4), (1, 2, 32, 32))
    assert a != c and b != c
    assert c == (1, 2, 3, 4) and (1, 2, 3, 4) == c
    assert c.with_tile_padding() == (1, 2, 32, 32) and (1, 2, 32, 32) == c.with_tile_padding()
    d = ttnn.Shape((1, 2, 32, 32))
    assert a != d and c != d and d == (1, 2, 32, 32) and d.with_tile_padding() == (1, 2, 32, 32)
    e = ttnn.Shape((1, 2, 3, 4), (1, 2, 32, 32))
    assert c == e and a != e and d != e
    f = ttnn.Shape((1, 2, 4, 4), (1, 2, 32, 32))
    assert all(x != f for x in (a, b, c, d, e)) and f == (1, 2, 4, 4)
    g = ttnn.Shape((2, 4, 4), (2, 32, 32))
    assert all(x != g for x in (a, b, c, d, e, f))
    assert g == (2, 4, 4) and g.with_tile_padding() == (2, 32, 32)


def test_shape_indexing_and_rank():
    s = ttnn.Shape((1, 2, 3, 4), (1, 2, 32, 32))
    assert len(s) == 4 and s.rank == 4 and s[-1] == 4 and s[-2] == 3 and tuple(s) == (1, 2, 3, 4)
    assert s[-2:] == (3, 4) and s[-2:].with_tile_padding() == (32, 32)
    assert "3[32]" in repr(s)
    with pytest.raises(RuntimeError):
        ttnn.Shape((1, 2), (1, 2, 3))


def test_names_match_the_reference_enums():
    # tt_eager/tensor/types.hpp:24-34: the integer values travel through the C ABI
    assert int(ttnn.bfloat16) == 0 and int(ttnn.float32) == 1 and int(ttnn.bfloat8_b) == 3 and int(ttnn.bfloat4_b) == 4
    assert int(ttnn.ROW_MAJOR_LAYOUT) == 0 and int(ttnn.TILE_LAYOUT) == 1 and ttnn.TILE_SIZE == 32
    assert tt_lib.tensor.DataType.BFLOAT8_B is ttnn.bfloat8_b and tt_lib.tensor.Layout.TILE is ttnn.TILE_LAYOUT
    assert ttnn.DRAM_MEMORY_CONFIG == tt_lib.tensor.MemoryConfig()


@pytest.mark.parametrize("dtype", [ttnn.bfloat8_b, ttnn.bfloat4_b])
def test_from_torch_block_float_argument_errors(dtype):
    with pytest.raises(RuntimeError, match="requires TILE_LAYOUT"):
        ttnn.from_torch(torch.zeros(32, 32), dtype=dtype, layout=ttnn.ROW_MAJOR_LAYOUT)
    with pytest.raises(RuntimeError, match="at least 2 dimensions"):
        ttnn.from_torch(torch.zeros(32), dtype=dtype, layout=ttnn.TILE_LAYOUT)
    with pytest.raises(RuntimeError, match="Rank 5 is not supported"):
        ttnn.from_torch(torch.zeros(1, 1, 1, 32, 32), dtype=dtype, layout=ttnn.TILE_LAYOUT)
    with pytest.raises(RuntimeError, match="must be of type"):
        ttnn.from_torch(torch.zeros(32, 32, dtype=torch.uint8), dtype=dtype, layout=ttnn.TILE_LAYOUT)
    with pytest.raises(RuntimeError, match="device must be specified"):
        ttnn.from_torch(torch.zeros(32, 32), dtype=dtype, layout=ttnn.TILE_LAYOUT, memory_config=ttnn.DRAM_MEMORY_CONFIG)


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-GPU error path")
def test_block_float_conversion_without_gpu_fails_loudly():
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ttnn.from_torch(torch.zeros(32, 32), dtype=ttnn.bfloat8_b, layout=ttnn.TILE_LAYOUT)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ttnn.open_device(0)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        tt_lib.tensor.Tensor(torch.zeros(1, 1, 32, 32), tt_lib.tensor.DataType.BFLOAT8_B)


def test_matmul_validation_on_host_tensors():
    a = ttnn.from_torch(torch.zeros(32, 32, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="layout TILE"):
        ttnn.matmul(a, a)
    with pytest.raises(RuntimeError, match="rank"):
        ttnn.matmul(ttnn.from_torch(torch.zeros(32, dtype=torch.bfloat16)), a)
    with pytest.raises(RuntimeError, match="must be of type"):
        ttnn.matmul(ttnn.from_torch(torch.zeros(32, 32, dtype=torch.float32)), a)


def _host_tile_tensor(shape, dtype=tt_lib.tensor.DataType.BFLOAT16):
    """A host tensor that claims TILE layout (no conversion needed to build it: only metadata is checked below)."""
    n = 1
    for s in shape:
        n *= s
    nbytes = {tt_lib.tensor.DataType.BFLOAT16: 2 * n, tt_lib.tensor.DataType.BFLOAT8_B: n // 1024 * 1088, tt_lib.tensor.DataType.BFLOAT4_B: n // 1024 * 576}[dtype]
    return tt_lib.tensor.Tensor(None, _raw=(torch.zeros(nbytes, dtype=torch.uint8), tuple(shape), tuple(shape), dtype, tt_lib.tensor.Layout.TILE, None))


def test_a_buffer_that_does_not_hold_its_shape_is_refused():
    """Kernels index a buffer by the tensor's shape: a raw buffer of another size never becomes a Tensor."""
    tile = tt_lib.tensor.Layout.TILE
    with pytest.raises(RuntimeError, match="the buffer holds 2048 bytes"):
        tt_lib.tensor.Tensor(None, _raw=(torch.zeros(2048, dtype=torch.uint8), (1, 1, 32, 64), (1, 1, 32, 64), tt_lib.tensor.DataType.BFLOAT16, tile, None))
    with pytest.raises(RuntimeError, match="whole tiles"):
        tt_lib.tensor.Tensor(None, _raw=(torch.zeros(544, dtype=torch.uint8), (1, 1, 16, 32), (1, 1, 16, 32), tt_lib.tensor.DataType.BFLOAT8_B,
                                         tt_lib.tensor.Layout.ROW_MAJOR, None))
    with pytest.raises(RuntimeError, match="larger without padding"):
        tt_lib.tensor.Tensor(None, _raw=(torch.zeros(2048, dtype=torch.uint8), (1, 1, 64, 32), (1, 1, 32, 32), tt_lib.tensor.DataType.BFLOAT16, tile, None))


def test_elementwise_argument_checks_need_no_gpu():
    """ttnn/ttnn/operations/binary.py:352-368: first operand a device tensor, second a tensor or a number."""
    host = _host_tile_tensor((32, 32))
    with pytest.raises(RuntimeError, match="must be on device"):
        ttnn.mul(host, host)
    with pytest.raises(TypeError, match="first argument"):
        ttnn.mul(torch.zeros(2), host)
    with pytest.raises(RuntimeError, match="must be on device"):
        ttnn.gelu(host)
    assert ttnn.multiply is ttnn.mul and ttnn.subtract is ttnn.sub


def test_falcon_matmul_shape_rules():
    """bmm_op.cpp:773-784: above 1024 rows falcon_dense_h_to_4h_matmul takes no fused activation and only the model's shapes."""
    gelu = [tt_lib.tensor.FusibleActivation.GELU, True]
    assert tt_lib.tensor.FusibleActivationWithParam(gelu).op_type == tt_lib.tensor.FusibleActivation.GELU
    assert int(tt_lib.tensor.FusibleActivation.GELU) == 2 and int(tt_lib.tensor.FusibleActivation.SILU) == 48     # UnaryOpType values
    a = _host_tile_tensor((1, 1, 2048, 64))
    w = _host_tile_tensor((1, 1, 64, 128), tt_lib.tensor.DataType.BFLOAT8_B)
    with pytest.raises(RuntimeError, match="fused_activation"):
        tt_lib.tensor.falcon_dense_h_to_4h_matmul(a, w, fused_activation=gelu)
    with pytest.raises(RuntimeError, match="Unsupported input shape"):
        tt_lib.tensor.falcon_dense_h_to_4h_matmul(a, w)
    with pytest.raises(RuntimeError, match="need to be on device"):
        tt_lib.tensor.falcon_dense_4h_to_h_matmul(_host_tile_tensor((1, 1, 32, 64)), w)


def test_as_tensor_and_clone_argument_checks():
    with pytest.raises(RuntimeError, match="must be of type"):
        ttnn.as_tensor(torch.zeros(4, 4, dtype=torch.float64))
    with pytest.raises(RuntimeError, match="must be of rank"):
        ttnn.as_tensor(torch.zeros(()))
    with pytest.raises(RuntimeError, match="on device"):
        ttnn.clone(_host_tile_tensor((32, 32)), None, ttnn.bfloat8_b)
    with pytest.raises(RuntimeError, match="Unsupported datatype conversion"):
        ttnn.to_layout(ttnn.from_torch(torch.zeros(32, 32, dtype=torch.bfloat16)), ttnn.TILE_LAYOUT, dtype=ttnn.bfloat8_b)
    with pytest.raises(RuntimeError, match="cannot slice"):
        ttnn.from_torch(torch.zeros(4, 4))[:2]


def test_tensix_only_objects_exist_and_are_inert():
    """Objects that model code constructs for a Tensix device — compute kernel configs, core grids, interleaved memory
    configs — exist with the reference's constructor arguments (tt_lib_bindings_tensor.cpp:325-348) and steer nothing."""
    import ttnn

    cfg = ttnn.WormholeComputeKernelConfig(math_fidelity=ttnn.MathFidelity.HiFi4, math_approx_mode=False, fp32_dest_acc_en=True, packer_l1_acc=True)
    assert (cfg.math_fidelity, cfg.math_approx_mode, cfg.fp32_dest_acc_en, cfg.packer_l1_acc) == (ttnn.MathFidelity.HiFi4, False, True, True)
    assert ttnn.GrayskullComputeKernelConfig(math_fidelity=ttnn.MathFidelity.LoFi).math_approx_mode is True
    with pytest.raises(TypeError):
        ttnn.WormholeComputeKernelConfig(ttnn.MathFidelity.HiFi4)          # keyword-only, as bound
    marker = object()
    assert ttnn.to_memory_config(marker, ttnn.DRAM_MEMORY_CONFIG) is marker and ttnn.to_memory_config(marker, ttnn.L1_MEMORY_CONFIG) is marker
    assert ttnn.CoreGrid(y=8, x=8).num_cores == 64
