"""The pybind11 layer over the C ABI: loads, mirrors sizes and argument errors on the CPU; on the GPU it produces the
same bytes as the ctypes layer (both end in the same C entry points)."""
import numpy as np
import pytest

from ttmi import capi, pybind, workloads


def test_module_loads_and_reports_sizes():
    m = pybind.module()
    assert m.version() == capi.lib().ttmi_version().decode()
    assert (m.BFLOAT16, m.FLOAT32, m.BFLOAT8_B, m.BFLOAT4_B, m.ROW_MAJOR, m.TILE) == (0, 1, 3, 4, 0, 1)
    assert m.tile_size(m.BFLOAT8_B) == 1088 and m.tile_size(m.BFLOAT4_B) == 576 and m.tile_size(99) == 0
    assert m.tiled_size_bytes(m.BFLOAT8_B, 2, 33, 65) == 2 * 2 * 3 * 1088
    assert m.matmul_workspace_bytes(1, 32, 4544, 18176, m.BFLOAT8_B) == capi.lib().ttmi_matmul_bfp_workspace_bytes(1, 32, 4544, 18176, 3)


def test_errors_become_runtime_errors():
    m = pybind.module()
    with pytest.raises(RuntimeError, match="null pointer"):
        m.from_torch(m.BFLOAT8_B, 0, m.FLOAT32, 1, 32, 32, 32, 1024, 0)
    with pytest.raises(RuntimeError, match="is not supported as activation function"):
        m.linear(0, m.TILE, 0, m.BFLOAT8_B, 1, 1, 32, 32, 32, activation="tanh")
    with pytest.raises(RuntimeError, match="Cannot use activation with batched input b"):
        m.linear(0, m.TILE, 0, m.BFLOAT8_B, 2, 2, 32, 32, 32, activation="relu")


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [capi.BFLOAT8_B, capi.BFLOAT4_B])
def test_same_bytes_as_the_ctypes_layer(fmt):
    import torch

    m = pybind.module()
    k, n, rows = 160, 96, 40
    w = torch.from_numpy(workloads.weights_f32(k, n, seed=5)).cuda()
    words = torch.empty(m.tiled_size_bytes(fmt, 1, k, n) // 4, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    m.from_torch(fmt, w.data_ptr(), m.FLOAT32, 1, k, n, n, k * n, words.data_ptr(), stream)
    assert torch.equal(words, capi.pack_tensor(fmt, w))
    back = torch.empty((k, n), dtype=torch.float32, device="cuda")
    m.to_torch(fmt, words.data_ptr(), 1, k, n, back.data_ptr(), m.FLOAT32, stream)
    assert torch.equal(back.view(torch.int32), capi.unpack_tensor(fmt, words, (k, n)).view(torch.int32))
    a_bits = workloads.activations_bf16(rows, k, seed=6)
    a = torch.from_numpy(a_bits.view(np.int16)).cuda().view(torch.bfloat16)
    bias = torch.randn(n, device="cuda").bfloat16()
    c = torch.empty((rows, n), dtype=torch.bfloat16, device="cuda")
    m.linear(a.data_ptr(), m.ROW_MAJOR, words.data_ptr(), fmt, 1, 1, rows, k, n, bias=bias.data_ptr(), activation="gelu",
             c=c.data_ptr(), c_layout=m.ROW_MAJOR, c_dtype=m.BFLOAT16, stream=stream)
    want = capi.matmul_bfp(a, capi.ROW_MAJOR, words, fmt, 1, 1, rows, k, n, bias=bias, activation=capi.ACT_GELU)[0]
    assert torch.equal(c.view(torch.int16), want.view(torch.int16))
