"""The TT-NN / tt_lib mirror on the GPU, in the shape of the reference's own tests:
tests/ttnn/unit_tests/test_to_and_from_torch.py, tests/ttnn/unit_tests/operations/test_matmul.py (test_sd_matmul),
tests/ttnn/unit_tests/operations/test_linear.py and tests/tt_eager/python_api_testing/unit_testing/misc/test_tensor.py,
with the CPU oracle as the bit-exact checker for every conversion."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def device():
    import ttnn

    dev = ttnn.open_device(0)
    yield dev
    ttnn.close_device(dev)


def _words(t):
    return t._buf.cpu().numpy().view(np.uint32)


@pytest.mark.parametrize("shape", [(7, 3), (1, 1, 7, 3), (2, 33, 65), (1, 2, 64, 96), (32, 32)])
@pytest.mark.parametrize("name", ["bfloat8_b", "bfloat4_b"])
@pytest.mark.parametrize("src_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("on_device", [False, True])
def test_to_and_from_torch_block_float(oracle, device, shape, name, src_dtype, on_device):
    import ttnn

    dtype = getattr(ttnn, name)
    torch.manual_seed(0)
    x = (torch.rand(shape, dtype=torch.float32) * 4 - 2).to(src_dtype)
    t = ttnn.from_torch(x, dtype=dtype, layout=ttnn.TILE_LAYOUT, device=device if on_device else None)
    assert t.dtype == dtype and t.layout == ttnn.TILE_LAYOUT
    assert t.shape == shape and t.shape.with_tile_padding() == shape[:-2] + ((shape[-2] + 31) // 32 * 32, (shape[-1] + 31) // 32 * 32)
    assert ttnn.is_tensor_storage_on_device(t) == on_device
    want = oracle.from_torch_bfp_tiles(int(dtype), x.float().numpy().reshape((-1,) + shape[-2:]))
    assert np.array_equal(_words(t), want)
    back = ttnn.to_torch(t)
    assert back.dtype == torch.float32 and tuple(back.shape) == shape
    ref = oracle.to_torch_bfp_tiles(int(dtype), want, (int(np.prod(shape[:-2])),) + shape[-2:]).reshape(shape)
    assert np.array_equal(back.numpy().view(np.uint32), ref.view(np.uint32))
    # the reference's own acceptance (test_to_and_from_torch.py:32-43)
    if name == "bfloat8_b":
        assert torch.allclose(x.float(), back, atol=2e-2)
    else:
        assert np.corrcoef(x.float().numpy().ravel(), back.numpy().ravel())[0, 1] > 0.9
    assert tuple(ttnn.to_torch(t, torch_rank=len(shape)).shape) == shape


def test_to_and_from_torch_bfloat16_layouts(device):
    import ttnn

    x = torch.rand((1, 1, 7, 3), dtype=torch.bfloat16)
    assert torch.equal(ttnn.to_torch(ttnn.from_torch(x)), x)
    t = ttnn.from_torch(x, layout=ttnn.TILE_LAYOUT, device=device)
    assert t.shape == (1, 1, 7, 3) and t.shape.with_tile_padding() == (1, 1, 32, 32)
    assert torch.equal(ttnn.to_torch(t), x)
    t = ttnn.to_layout(ttnn.from_device(t), ttnn.ROW_MAJOR_LAYOUT)
    assert torch.equal(ttnn.to_torch(t), x)


@pytest.mark.parametrize("batch_size, channel_a, channel_b, m, k, n", [
    (1, 2, 1, 64, 320, 160), (2, 8, 8, 128, 64, 96), (1, 1, 1, 32, 4544, 4672 // 4), (1, 2, 1, 256, 1280, 512)])
@pytest.mark.parametrize("name", ["bfloat8_b", "bfloat4_b"])
def test_sd_matmul(oracle, device, batch_size, channel_a, channel_b, m, k, n, name):
    """test_matmul.py:561-620: both operands block-float; bit-level check of the operands, bound + PCC on the product."""
    import ttnn

    dtype = getattr(ttnn, name)
    torch.manual_seed(0)
    ta = torch.randn((batch_size, channel_a, m, k), dtype=torch.bfloat16)
    tb = torch.randn((batch_size, channel_b, k, n), dtype=torch.bfloat16)
    a = ttnn.from_torch(ta, layout=ttnn.TILE_LAYOUT, device=device, dtype=dtype)
    b = ttnn.from_torch(tb, layout=ttnn.TILE_LAYOUT, device=device, dtype=dtype)
    out = ttnn.matmul(a, b, core_grid=ttnn.CoreGrid(x=8, y=8), dtype=ttnn.bfloat16)
    assert out.shape == (batch_size, channel_a, m, n) and out.layout == ttnn.TILE_LAYOUT and out.dtype == ttnn.bfloat16
    got = ttnn.to_torch(out).double()
    if m == 32 and name == "bfloat8_b":
        # one band of rows: the kernel that streams the weights took the packed activations as they are; expanding them
        # first gives the same bits
        import tt_lib

        a16 = tt_lib.tensor.typecast(a, ttnn.bfloat16)
        assert torch.equal(ttnn.to_torch(ttnn.matmul(a16, b, dtype=ttnn.bfloat16)), ttnn.to_torch(out))
    # the quantised operands come from the CPU oracle (the host sequences of from_torch and to_torch), not from this library
    quantise = lambda t: torch.from_numpy(oracle.to_torch_bfp_tiles(int(dtype), oracle.from_torch_bfp_tiles(int(dtype), t.float().numpy()), tuple(t.shape))).double()
    aq, bq = quantise(ta), quantise(tb)
    assert torch.equal(ttnn.to_torch(a).double(), aq) and torch.equal(ttnn.to_torch(b).double(), bq)
    ref = aq @ bq
    bound = 2.0 ** -8 * ref.abs() + 2.0 * k * 2.0 ** -24 * (aq.abs() @ bq.abs()) + 1e-30
    assert bool(((got - ref).abs() <= bound).all())
    assert np.corrcoef(got.numpy().ravel(), ref.numpy().ravel())[0, 1] >= 0.9999
    # the reference's acceptance against the unquantised product (pcc 0.94 for bfloat8_b)
    pcc = np.corrcoef(got.numpy().ravel(), (ta.double() @ tb.double()).numpy().ravel())[0, 1]
    assert pcc >= (0.94 if name == "bfloat8_b" else 0.9)
    # default output dtype follows input a, packed by the same rules as a host pack of the bf16 result
    out_q = ttnn.matmul(a, b)
    assert out_q.dtype == dtype
    tiles = out._buf.float().cpu().numpy().reshape(-1)
    assert np.array_equal(_words(out_q), oracle.pack_fp32_vec_as_bfp_tiles(int(dtype), tiles, row_major_input=False))
    back = ttnn.to_torch(out_q).double()
    assert np.corrcoef(back.numpy().ravel(), ref.numpy().ravel())[0, 1] >= (0.999 if name == "bfloat8_b" else 0.97)


@pytest.mark.parametrize("activation", [None, "relu", "gelu", "silu"])
@pytest.mark.parametrize("use_bias", [False, True])
def test_linear_bias_activation(device, activation, use_bias):
    """test_linear.py: bias is a [1, N] row broadcast over rows; activation fused after it."""
    import ttnn

    torch.manual_seed(1)
    m, k, n = 64, 256, 192
    ta = torch.randn((1, m, k), dtype=torch.bfloat16)
    tb = torch.randn((k, n), dtype=torch.bfloat16) * 0.1
    tbias = torch.randn((1, n), dtype=torch.bfloat16)
    a = ttnn.from_torch(ta, layout=ttnn.TILE_LAYOUT, device=device)
    b = ttnn.from_torch(tb, layout=ttnn.TILE_LAYOUT, device=device, dtype=ttnn.bfloat8_b)
    bias = ttnn.from_torch(tbias, layout=ttnn.TILE_LAYOUT, device=device) if use_bias else None
    out = ttnn.linear(a, b, bias=bias, activation=activation)
    assert out.shape == (1, m, n)
    ref = ta.double() @ ttnn.to_torch(b).double()
    if use_bias:
        ref = ref + tbias.double()
    ref = {None: lambda v: v, "relu": torch.relu, "gelu": torch.nn.functional.gelu, "silu": torch.nn.functional.silu}[activation](ref)
    got = ttnn.to_torch(out).double()
    assert torch.allclose(got, ref, rtol=2 ** -7, atol=2e-2)
    assert np.corrcoef(got.numpy().ravel(), ref.numpy().ravel())[0, 1] >= 0.9999


def test_matmul_errors(device):
    import ttnn

    a = ttnn.from_torch(torch.zeros((32, 64), dtype=torch.bfloat16), layout=ttnn.TILE_LAYOUT, device=device)
    b = ttnn.from_torch(torch.zeros((32, 64), dtype=torch.bfloat16), layout=ttnn.TILE_LAYOUT, device=device, dtype=ttnn.bfloat8_b)
    with pytest.raises(RuntimeError, match="The width of the first tensor must be equal to the height of the second tensor"):
        ttnn.matmul(a, b)
    with pytest.raises(RuntimeError, match="must be on device"):
        ttnn.matmul(ttnn.from_device(a), b)
    b2 = ttnn.from_torch(torch.zeros((2, 64, 32), dtype=torch.bfloat16), layout=ttnn.TILE_LAYOUT, device=device, dtype=ttnn.bfloat8_b)
    a2 = ttnn.from_torch(torch.zeros((2, 32, 64), dtype=torch.bfloat16), layout=ttnn.TILE_LAYOUT, device=device)
    with pytest.raises(RuntimeError, match="Cannot use activation with batched input b"):
        ttnn.linear(a2, b2, activation="relu")
    with pytest.raises(RuntimeError, match="is not supported as activation function"):
        ttnn.linear(a2, b2, activation="tanh")
    assert (a2 @ b2).shape == (2, 32, 32)


def test_matmul_of_two_bfloat16_tensors(device):
    """ttnn.matmul / ttnn.linear with two bf16 operands (matmul.hpp:39-42): the surface is the same, the weights take the
    re-layout path of ttmi_matmul_bf16."""
    import ttnn

    torch.manual_seed(11)
    x = torch.randn((2, 64, 96), dtype=torch.bfloat16)
    w = torch.randn((96, 160), dtype=torch.bfloat16)
    bias = torch.randn((1, 160), dtype=torch.bfloat16)
    tx = ttnn.from_torch(x, layout=ttnn.TILE_LAYOUT, device=device)
    tw = ttnn.from_torch(w, layout=ttnn.TILE_LAYOUT, device=device)
    tb = ttnn.from_torch(bias, layout=ttnn.TILE_LAYOUT, device=device)
    got = ttnn.to_torch(ttnn.matmul(tx, tw)).float()
    ref = x.double() @ w.double()
    assert got.shape == (2, 64, 160)
    assert torch.allclose(got.double(), ref, rtol=2 ** -7, atol=2e-2)
    got = ttnn.to_torch(ttnn.linear(tx, tw, bias=tb, activation="relu")).float()
    assert torch.allclose(got.double(), torch.relu(ref + bias.double()), rtol=2 ** -7, atol=2e-2)


@pytest.mark.parametrize("name", ["BFLOAT8_B", "BFLOAT4_B"])
@pytest.mark.parametrize("shape", [(1, 1, 32, 32), (2, 3, 64, 96)])
def test_tt_lib_tensor_conversion(oracle, shape, name):
    """test_tensor.py:28-78: Tensor(torch, dtype) packs 1024-element runs, .to(TILE) re-packs the tilized data,
    to_torch returns float32, block-float storage is OWNED."""
    import tt_lib as ttl

    dtype = getattr(ttl.tensor.DataType, name)
    torch.manual_seed(2)
    x = torch.rand(shape, dtype=torch.float32) * 6 - 3
    t = ttl.tensor.Tensor(x, dtype)
    assert t.storage_type() == ttl.tensor.StorageType.OWNED and t.get_layout() == ttl.tensor.Layout.ROW_MAJOR
    assert tuple(t.get_legacy_shape()) == shape and t.get_dtype() == dtype
    flat = x.numpy().reshape(-1)
    want = oracle.pack_fp32_vec_as_bfp_tiles(int(dtype), flat, row_major_input=False)
    assert np.array_equal(_words(t), want)
    back = t.to_torch()
    assert back.dtype == torch.float32
    assert np.array_equal(back.numpy().reshape(-1).view(np.uint32),
                          oracle.unpack_bfp_tiles_into_float_vec(int(dtype), want, row_major_output=False).view(np.uint32))
    tiled = t.to(ttl.tensor.Layout.TILE)
    assert np.array_equal(_words(tiled), oracle.from_torch_bfp_tiles(int(dtype), x.numpy().reshape((-1,) + shape[-2:])))
    rm = tiled.to(ttl.tensor.Layout.ROW_MAJOR)
    assert np.array_equal(rm.to_torch().numpy().view(np.uint32),
                          oracle.to_torch_bfp_tiles(int(dtype), _words(tiled), (shape[0] * shape[1],) + shape[-2:]).reshape(shape).view(np.uint32))


def test_tt_lib_matmul_and_bmm(device):
    import tt_lib as ttl

    torch.manual_seed(3)
    a = torch.randn((2, 2, 64, 128), dtype=torch.bfloat16)
    w = torch.randn((1, 1, 128, 96), dtype=torch.float32)
    ta = ttl.tensor.Tensor(a, ttl.tensor.DataType.BFLOAT16).to(ttl.tensor.Layout.TILE).to(device)
    tw = ttl.tensor.Tensor(w, ttl.tensor.DataType.BFLOAT8_B).to(ttl.tensor.Layout.TILE).to(device)
    out = ttl.tensor.matmul(ta, tw)
    assert tuple(out.get_legacy_shape()) == (2, 2, 64, 96)
    wq = tw.cpu().to(ttl.tensor.Layout.ROW_MAJOR).to_torch().double()
    ref = a.double() @ wq
    got = out.cpu().to(ttl.tensor.Layout.ROW_MAJOR).to_torch().double()
    assert torch.allclose(got, ref, rtol=2 ** -7, atol=1e-2)
    wb = torch.randn((2, 2, 128, 96), dtype=torch.float32)
    twb = ttl.tensor.Tensor(wb, ttl.tensor.DataType.BFLOAT4_B).to(ttl.tensor.Layout.TILE).to(device)
    outb = ttl.tensor.bmm(ta, twb)
    refb = a.double() @ twb.cpu().to(ttl.tensor.Layout.ROW_MAJOR).to_torch().double()
    assert torch.allclose(outb.cpu().to(ttl.tensor.Layout.ROW_MAJOR).to_torch().double(), refb, rtol=2 ** -7, atol=1e-2)
    with pytest.raises(RuntimeError, match="BCMK\\*11KN"):
        ttl.tensor.matmul(ta, twb)
    with pytest.raises(RuntimeError, match="need to be on device"):
        ttl.tensor.matmul(ta.cpu(), tw)
    out2 = ttl.operations.primary.matmul(ta, tw)
    assert torch.equal(out2.cpu().to(ttl.tensor.Layout.ROW_MAJOR).to_torch(), out.cpu().to(ttl.tensor.Layout.ROW_MAJOR).to_torch())


@pytest.mark.parametrize("batch_size,m_size,k_size,n_size", [(1, 31, 1024, 1023), (3, 63, 512, 2047)])
def test_matmul_by_passing_in_1d_systolic_array_program_config(device, batch_size, m_size, k_size, n_size):
    """tests/ttnn/unit_tests/operations/test_matmul.py:460-486: ttnn.create_matmul_1d_systolic_array_program_config from the
    padded shapes, passed to ttnn.matmul; here also with block-float weights and with an activation carried by the config."""
    import ttnn

    torch.manual_seed(0)
    ta = torch.randn((batch_size, m_size, k_size), dtype=torch.bfloat16)
    tb = torch.randn((k_size, n_size), dtype=torch.bfloat16)
    a = ttnn.from_torch(ta, layout=ttnn.TILE_LAYOUT, device=device)
    for dtype in (ttnn.bfloat16, ttnn.bfloat8_b):
        b = ttnn.from_torch(tb, layout=ttnn.TILE_LAYOUT, device=device, dtype=dtype)
        config = ttnn.create_matmul_1d_systolic_array_program_config(
            input_shape_a=a.shape.with_tile_padding(), input_shape_b=b.shape.with_tile_padding(), core_grid=ttnn.CoreGrid(y=8, x=8))
        assert config.fused_activation is None and config.fuse_batch is True
        out = ttnn.to_torch(ttnn.matmul(a, b, program_config=config))
        ref = ta.double() @ ttnn.to_torch(b).double()
        assert out.shape == (batch_size, m_size, n_size)
        assert np.corrcoef(out.double().numpy().ravel(), ref.numpy().ravel())[0, 1] >= 0.9999
        relu = ttnn.create_matmul_1d_systolic_array_program_config(
            input_shape_a=a.shape.with_tile_padding(), input_shape_b=b.shape.with_tile_padding(), activation="relu")
        assert torch.equal(ttnn.to_torch(ttnn.matmul(a, b, program_config=relu)), torch.relu(out))
    with pytest.raises(RuntimeError):
        ttnn.create_matmul_1d_systolic_array_program_config(input_shape_a=(32, 64), input_shape_b=(96, 32))
    with pytest.raises(RuntimeError):
        ttnn.create_matmul_1d_systolic_array_program_config(input_shape_a=(32, 64), input_shape_b=(64, 32), activation="tanh")


def test_primary_matmul_1d_with_program_config_and_block_float_chain(device):
    """tt_lib.operations.primary.matmul_1d (module.hpp:373-406) as Falcon-40B's MLP issues it
    (models/demos/falcon40b/tt/falcon_mlp.py:97-135): a 1D program config that carries the fused GELU, a BFLOAT8_B output
    of the first GEMM feeding the second as its activations.  The program config objects are plain holders (keyword-only
    constructors as in module.hpp:53-122); the fused activation is honoured."""
    import tt_lib as ttl

    P = ttl.operations.primary
    torch.manual_seed(9)
    h, f = 256, 1024
    x = torch.randn((1, 1, 32, h), dtype=torch.bfloat16) * 0.5
    w1, w2 = torch.randn((1, 1, h, f)) * 0.05, torch.randn((1, 1, f, h)) * 0.05
    tx = ttl.tensor.Tensor(x, ttl.tensor.DataType.BFLOAT16).to(ttl.tensor.Layout.TILE).to(device)
    t1 = ttl.tensor.Tensor(w1, ttl.tensor.DataType.BFLOAT8_B).to(ttl.tensor.Layout.TILE).to(device)
    t2 = ttl.tensor.Tensor(w2, ttl.tensor.DataType.BFLOAT8_B).to(ttl.tensor.Layout.TILE).to(device)
    config = P.MatmulMultiCoreReuseMultiCast1DProgramConfig(
        compute_with_storage_grid_size=(8, 4), in0_block_w=2, out_subblock_h=1, out_subblock_w=4, per_core_M=1, per_core_N=1,
        fuse_batch=True, fused_activation=[ttl.tensor.FusibleActivation.GELU, True], mcast_in0=True)
    assert "in0_block_w=2" in repr(config)
    with pytest.raises(TypeError):
        P.MatmulMultiCoreReuseMultiCast1DProgramConfig(in0_block_w=2)
    hidden = P.matmul_1d(tx, t1, program_config=config, output_dtype=ttl.tensor.DataType.BFLOAT8_B)
    assert hidden.get_dtype() == ttl.tensor.DataType.BFLOAT8_B and tuple(hidden.get_legacy_shape()) == (1, 1, 32, f)
    out = P.matmul_1d(hidden, t2, output_dtype=ttl.tensor.DataType.BFLOAT16)
    back = lambda t: t.cpu().to(ttl.tensor.Layout.ROW_MAJOR).to_torch().double()
    h_ref = torch.nn.functional.gelu(x.double() @ back(t1))
    assert np.corrcoef(back(hidden).numpy().ravel(), h_ref.numpy().ravel())[0, 1] >= 0.999
    ref = back(hidden) @ back(t2)                                  # from the quantised intermediate the device holds
    got = back(out)
    bound = 2.0 ** -8 * ref.abs() + 2.0 * f * 2.0 ** -24 * (back(hidden).abs() @ (5.0 * back(t2).abs().amax(dim=-1, keepdim=True).expand_as(back(t2)))) + 1e-30
    assert bool(((got - ref).abs() <= bound).all())
    # the same chain op by op with a bf16 intermediate typecast to BFLOAT8_B gives the same hidden tensor
    plain = P.matmul(tx, t1, program_config=config)
    assert torch.equal(back(ttl.tensor.typecast(plain, ttl.tensor.DataType.BFLOAT8_B)), back(hidden))
    with pytest.raises(RuntimeError, match="not supported as activation"):
        P.matmul(tx, t1, activation="tanh")


@pytest.mark.parametrize("m", [32, 64, 96, 160, 544])        # every GEMM kernel: one band, two bands, three bands, tiled, expanded
def test_untilize_out_gives_the_tile_result_row_major(device, m):
    """bmm_op.cpp:1069: with untilize_out the output tensor is ROW_MAJOR; :536-538, :865-867: bfloat16 only.  The values are
    those of the TILE output, untilized, bit for bit."""
    import tt_lib as ttl

    torch.manual_seed(5)
    a = torch.randn((1, 2, m, 256), dtype=torch.bfloat16)
    w = torch.randn((1, 1, 256, 192), dtype=torch.float32)
    ta = ttl.tensor.Tensor(a, ttl.tensor.DataType.BFLOAT16).to(ttl.tensor.Layout.TILE).to(device)
    tw = ttl.tensor.Tensor(w, ttl.tensor.DataType.BFLOAT8_B).to(ttl.tensor.Layout.TILE).to(device)
    tiles = ttl.tensor.matmul(ta, tw)
    for rows in (ttl.tensor.matmul(ta, tw, untilize_out=True), ttl.operations.primary.matmul(ta, tw, untilize_out=True)):
        assert rows.get_layout() == ttl.tensor.Layout.ROW_MAJOR and tuple(rows.get_legacy_shape()) == (1, 2, m, 192)
        assert rows.get_dtype() == ttl.tensor.DataType.BFLOAT16
        assert torch.equal(rows.cpu().to_torch().view(torch.int16), tiles.cpu().to(ttl.tensor.Layout.ROW_MAJOR).to_torch().view(torch.int16))
    twb = ttl.tensor.Tensor(torch.randn((1, 2, 256, 192)), ttl.tensor.DataType.BFLOAT8_B).to(ttl.tensor.Layout.TILE).to(device)
    rows = ttl.tensor.bmm(ta, twb, untilize_out=True)
    assert torch.equal(rows.cpu().to_torch().view(torch.int16), ttl.tensor.bmm(ta, twb).cpu().to(ttl.tensor.Layout.ROW_MAJOR).to_torch().view(torch.int16))
    with pytest.raises(RuntimeError, match="output_dtype == DataType::BFLOAT16"):
        ttl.operations.primary.matmul(ta, tw, output_dtype=ttl.tensor.DataType.BFLOAT8_B, untilize_out=True)
